// cos/sin table builder: out[p, i] = cos(p * inv[i]), out[p, R/2 + i] = sin(p * inv[i]).
// inv follows lazy_attn/lazy/model_executor/rope/cos_sin.py:41-58 (plain, or Llama-3
// wavelength smoothing).  The angle p*inv is formed and reduced in float64 so that rows
// at large positions are as accurate as rows near zero; the result is rounded once to the
// table's element type.
#include "common.hpp"

namespace lazyattn {

template <typename T>
__global__ void __launch_bounds__(256)
cos_sin_table_kernel(T *out, int64_t row_stride, int max_position, int rotary_dim, double base,
                     int rope_type, double factor, double low, double high, int orig_max) {
    const int half = rotary_dim / 2;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)max_position * half) return;
    const int i = (int)(idx % half);
    const int64_t pos = idx / half;
    double inv = 1.0 / pow(base, (2.0 * i) / rotary_dim);           // cos_sin.py:41-43
    if (rope_type == 1) {                                           // cos_sin.py:44-58
        const double two_pi = 6.283185307179586476925286766559;
        const double wave_len = two_pi / inv;
        const double low_wl = orig_max / low, high_wl = orig_max / high;
        if (wave_len < high_wl) {
        } else if (wave_len > low_wl) {
            inv = inv / factor;
        } else {
            const double smooth = (orig_max / wave_len - low) / (high - low);
            inv = (1.0 - smooth) * inv / factor + smooth * inv;
        }
    }
    const double ang = (double)pos * inv;
    out[pos * row_stride + i] = from_f32<T>((float)cos(ang));
    out[pos * row_stride + half + i] = from_f32<T>((float)sin(ang));
}

int launch_cos_sin_table(void *out, int out_dtype, int64_t row_stride, int max_position,
                         int rotary_dim, double base, int rope_type, double factor, double low,
                         double high, int orig_max, hipStream_t stream) {
    const int64_t n = (int64_t)max_position * (rotary_dim / 2);
    if (n <= 0) return LAZYATTN_OK;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    switch (out_dtype) {
        case LAZYATTN_F32:
            hipLaunchKernelGGL(cos_sin_table_kernel<float>, grid, block, 0, stream, (float *)out, row_stride,
                               max_position, rotary_dim, base, rope_type, factor, low, high, orig_max);
            break;
        case LAZYATTN_BF16:
            hipLaunchKernelGGL(cos_sin_table_kernel<bf16_t>, grid, block, 0, stream, (bf16_t *)out, row_stride,
                               max_position, rotary_dim, base, rope_type, factor, low, high, orig_max);
            break;
        case LAZYATTN_F16:
            hipLaunchKernelGGL(cos_sin_table_kernel<f16_t>, grid, block, 0, stream, (f16_t *)out, row_stride,
                               max_position, rotary_dim, base, rope_type, factor, low, high, orig_max);
            break;
        default: return LAZYATTN_E_DTYPE;
    }
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

// packed[h][c][p][e] = table[p, h*R/2 + c*8 + e]: one thread moves one 8-element chunk
template <typename T>
__global__ void __launch_bounds__(256)
pack_cos_sin_kernel(const T *table, T *packed, int64_t row_stride, int rows, int rotary_dim) {
    const int chunks = rotary_dim / 8;               // per row: R/16 cos chunks then R/16 sin chunks
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)rows * chunks) return;
    const int hc = (int)(idx % chunks);              // h * (R/16) + c
    const int64_t pos = idx / chunks;
    const T *src = table + pos * row_stride + hc * 8;
    T *dst = packed + ((int64_t)hc * rows + pos) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) dst[e] = src[e];
}

int launch_pack_cos_sin(const void *table, void *packed, int dtype, int64_t row_stride, int rows,
                        int rotary_dim, hipStream_t stream) {
    const int64_t n = (int64_t)rows * (rotary_dim / 8);
    if (n <= 0) return LAZYATTN_OK;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    switch (dtype) {
        case LAZYATTN_F32:
            hipLaunchKernelGGL(pack_cos_sin_kernel<float>, grid, block, 0, stream, (const float *)table,
                               (float *)packed, row_stride, rows, rotary_dim);
            break;
        case LAZYATTN_BF16:
        case LAZYATTN_F16:
            hipLaunchKernelGGL(pack_cos_sin_kernel<uint16_t>, grid, block, 0, stream, (const uint16_t *)table,
                               (uint16_t *)packed, row_stride, rows, rotary_dim);
            break;
        default: return LAZYATTN_E_DTYPE;
    }
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

}  // namespace lazyattn
