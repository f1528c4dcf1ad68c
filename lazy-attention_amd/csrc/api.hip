// C ABI: argument checks and kernel selection.  Nothing here allocates or synchronises.
#include "common.hpp"
#include <atomic>
#include <mutex>

namespace lazyattn {
int launch_prefill_generic(const lazyattn_prefill_params &p, int decode, hipStream_t stream);
int launch_prefill_mfma(const lazyattn_prefill_params &p, hipStream_t stream);
bool mfma_supports(const lazyattn_prefill_params &p);
const char *mfma_unsupported_reason(const lazyattn_prefill_params &p);
void mfma_choices(const lazyattn_prefill_params &p, int *waves, int *splits);
size_t mfma_workspace_bytes(const lazyattn_prefill_params &p);
int launch_decode_mfma(const lazyattn_prefill_params &p, hipStream_t stream);
bool decode_mfma_supports(const lazyattn_prefill_params &p);
size_t decode_workspace_bytes(const lazyattn_prefill_params &p);
int launch_rope_cache_write(const lazyattn_rope_write_params &p, hipStream_t stream);
int launch_rotation_metadata(const int32_t *doc_lens, const int32_t *doc_lens_padded, const int32_t *doc_start, int batch,
                             int block_size, int zero_offsets, int32_t *q_offset, int32_t *q_mask, int64_t row_stride,
                             int row_len, int32_t *max_offset, hipStream_t stream);
int launch_block_reposition(const lazyattn_reposition_params &p, hipStream_t stream);
int launch_pack_block_table(const int32_t *block_table, int64_t bt_stride, const int32_t *q_offset, const int32_t *q_mask,
                            int64_t row_stride, const int32_t *rows, int n_rows, int row_len, int64_t *packed,
                            int64_t packed_stride, hipStream_t stream);
int launch_cos_sin_table(void *out, int out_dtype, int64_t row_stride, int max_position,
                         int rotary_dim, double base, int rope_type, double factor, double low,
                         double high, int orig_max, hipStream_t stream);
int launch_pack_cos_sin(const void *table, void *packed, int dtype, int64_t row_stride, int rows,
                        int rotary_dim, hipStream_t stream);
}  // namespace lazyattn

using namespace lazyattn;

int lazyattn::device_cus() {
    constexpr int MAX_DEV = 64, FALLBACK = 256;
    static std::atomic<int> cus[MAX_DEV];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) { (void)hipGetLastError(); return FALLBACK; }
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return FALLBACK;
    }
    cus[dev].store(n, std::memory_order_relaxed);
    return n;
}

static int elem_bytes(int dt) {
    switch (dt) {
        case LAZYATTN_F32: return 4;
        case LAZYATTN_BF16:
        case LAZYATTN_F16: return 2;
        case LAZYATTN_FP8_E4M3:
        case LAZYATTN_FP8_E5M2: return 1;
        default: return 0;
    }
}

static int check_common(const lazyattn_prefill_params *p, bool decode) {
    if (!p) return LAZYATTN_E_NULL;
    if (!p->q || !p->o || !p->k_cache || !p->v_cache || !p->b_start_loc || !p->b_seq_len) return LAZYATTN_E_NULL;
    // the q_len == 1 entry takes the packed table in place of the three int32 tables, and frequencies in place of the table
    const bool packed = decode && p->packed_block_table;
    if (!p->block_table && !packed) return LAZYATTN_E_NULL;
    if (!p->cos_sin_cache && !(decode && p->rope_freqs)) return LAZYATTN_E_NULL;
    if (!decode && (!p->k || !p->v)) return LAZYATTN_E_NULL;
    if (p->batch < 0 || p->num_q_heads <= 0 || p->num_kv_heads <= 0 || p->head_dim <= 0 ||
        p->block_size <= 0 || p->x <= 0)
        return LAZYATTN_E_SHAPE;
    if (p->num_q_heads % p->num_kv_heads) return LAZYATTN_E_SHAPE;
    if (p->head_dim % 2 || p->head_dim % p->x || p->head_dim > 256) return LAZYATTN_E_SHAPE;
    if (p->rotary_dim != p->head_dim) return LAZYATTN_E_UNSUPPORTED;
    if (p->index_bits != 32 && p->index_bits != 64) return LAZYATTN_E_DTYPE;
    if (p->dtype != LAZYATTN_F32 && p->dtype != LAZYATTN_BF16 && p->dtype != LAZYATTN_F16)
        return LAZYATTN_E_DTYPE;
    const bool fp8 = p->cache_dtype == LAZYATTN_FP8_E4M3 || p->cache_dtype == LAZYATTN_FP8_E5M2;
    if (!fp8 && p->cache_dtype != p->dtype) return LAZYATTN_E_DTYPE;
    if (fp8 && (!p->k_scale || !p->v_scale)) return LAZYATTN_E_NULL;
    if (p->table_dtype != p->dtype && p->table_dtype != LAZYATTN_F32) return LAZYATTN_E_DTYPE;
    if (p->pos_mode < LAZYATTN_POS_NATURAL || p->pos_mode > LAZYATTN_POS_BLOCK_UNIFORM)
        return LAZYATTN_E_UNSUPPORTED;
    if (p->pos_mode != LAZYATTN_POS_NATURAL && !p->q_offset && !packed) return LAZYATTN_E_NULL;
    (void)elem_bytes;
    return LAZYATTN_OK;
}

extern "C" size_t lazyattn_prefill_workspace_bytes(const lazyattn_prefill_params *p) {
    if (!p || check_common(p, false) != LAZYATTN_OK) return 0;
    if (p->kernel == LAZYATTN_KERNEL_GENERIC) return 0;
    if (!mfma_supports(*p)) return 0;
    return mfma_workspace_bytes(*p);
}

extern "C" int lazyattn_prefix_prefill(const lazyattn_prefill_params *p, void *stream) {
    int rc = check_common(p, false);
    if (rc != LAZYATTN_OK) return rc;
    if (p->batch == 0 || p->max_q_len <= 0) return LAZYATTN_OK;
    hipStream_t s = (hipStream_t)stream;
    int kernel = p->kernel;
    if (kernel == LAZYATTN_KERNEL_AUTO)
        kernel = mfma_supports(*p) ? LAZYATTN_KERNEL_MFMA : LAZYATTN_KERNEL_GENERIC;
    if (kernel == LAZYATTN_KERNEL_MFMA || kernel == LAZYATTN_KERNEL_MFMA4 || kernel == LAZYATTN_KERNEL_MFMA8) {
        if (!mfma_supports(*p)) return LAZYATTN_E_UNSUPPORTED;
        return launch_prefill_mfma(*p, s);
    }
    if (kernel == LAZYATTN_KERNEL_GENERIC) return launch_prefill_generic(*p, 0, s);
    return LAZYATTN_E_UNSUPPORTED;
}

extern "C" int lazyattn_prefill_kernel_for(const lazyattn_prefill_params *p, int32_t *num_splits, const char **reason) {
    if (num_splits) *num_splits = 1;
    if (reason) *reason = nullptr;
    int rc = check_common(p, false);
    if (rc != LAZYATTN_OK) return rc;
    const char *why = mfma_unsupported_reason(*p);
    int kernel = p->kernel;
    if (kernel == LAZYATTN_KERNEL_AUTO) kernel = why ? LAZYATTN_KERNEL_GENERIC : LAZYATTN_KERNEL_MFMA;
    if (kernel == LAZYATTN_KERNEL_GENERIC) {
        if (reason) *reason = p->kernel == LAZYATTN_KERNEL_GENERIC ? "the call asks for it" : why;
        return LAZYATTN_KERNEL_GENERIC;
    }
    if (kernel != LAZYATTN_KERNEL_MFMA && kernel != LAZYATTN_KERNEL_MFMA4 && kernel != LAZYATTN_KERNEL_MFMA8) return LAZYATTN_E_UNSUPPORTED;
    if (why) {
        if (reason) *reason = why;
        return LAZYATTN_E_UNSUPPORTED;
    }
    int waves = 4, splits = 1;
    mfma_choices(*p, &waves, &splits);
    if (num_splits) *num_splits = splits;
    return waves == 8 ? LAZYATTN_KERNEL_MFMA8 : LAZYATTN_KERNEL_MFMA4;
}

extern "C" int lazyattn_paged_decode_kernel_for(const lazyattn_prefill_params *p) {
    int rc = check_common(p, true);
    if (rc != LAZYATTN_OK) return rc;
    if (p->pos_mode == LAZYATTN_POS_OFFSET) return LAZYATTN_E_UNSUPPORTED;
    if (p->kernel != LAZYATTN_KERNEL_GENERIC && decode_mfma_supports(*p)) return LAZYATTN_KERNEL_MFMA;
    if (p->packed_block_table || p->rope_freqs) return LAZYATTN_E_UNSUPPORTED;
    if (p->kernel != LAZYATTN_KERNEL_AUTO && p->kernel != LAZYATTN_KERNEL_GENERIC) return LAZYATTN_E_UNSUPPORTED;
    return LAZYATTN_KERNEL_GENERIC;
}

// ---- the prefill call for callers that may not allocate ----
// Split-KV partials of lazyattn_prefix_prefill_static_scratch() live in this array instead of a caller-provided
// workspace.  One copy per GPU the library runs on, held until the process ends.  In host code the array's name
// is only a handle: its device address is asked for once per device (with that device current) and kept.
namespace {
constexpr size_t STATIC_SCRATCH_BYTES = 32u << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void *scratch_ptr[MAX_DEVICES] = {};

int static_scratch_address(void **out) {
    // (the current device: the kernels are launched on it, so this is the copy of the array they will see)
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return LAZYATTN_E_LAUNCH;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return LAZYATTN_E_LAUNCH;
        scratch_ptr[dev] = ptr;
    }
    *out = scratch_ptr[dev];
    return LAZYATTN_OK;
}
}  // namespace

extern "C" size_t lazyattn_static_scratch_bytes(void) { return STATIC_SCRATCH_BYTES; }

extern "C" int lazyattn_static_scratch_prepare(void) {
    void *ptr = nullptr;
    return static_scratch_address(&ptr);
}

extern "C" int lazyattn_prefix_prefill_static_scratch(const lazyattn_prefill_params *p, void *stream) {
    int rc = check_common(p, false);
    if (rc != LAZYATTN_OK) return rc;
    const size_t need = lazyattn_prefill_workspace_bytes(p);
    if (need > STATIC_SCRATCH_BYTES) return LAZYATTN_E_SCRATCH_LIMIT;
    lazyattn_prefill_params q = *p;
    q.workspace = nullptr;
    q.workspace_bytes = 0;
    if (need > 0) {
        void *ptr = nullptr;
        rc = static_scratch_address(&ptr);
        if (rc != LAZYATTN_OK) return rc;
        q.workspace = ptr;                      // the kernels take the address as they take a caller's workspace
        q.workspace_bytes = (int64_t)STATIC_SCRATCH_BYTES;
    }
    return lazyattn_prefix_prefill(&q, stream);
}

extern "C" int lazyattn_paged_decode_rotary(const lazyattn_prefill_params *p, void *stream) {
    int rc = check_common(p, true);
    if (rc != LAZYATTN_OK) return rc;
    if (p->pos_mode == LAZYATTN_POS_OFFSET) return LAZYATTN_E_UNSUPPORTED;
    if (p->batch == 0) return LAZYATTN_OK;
    if (p->kernel != LAZYATTN_KERNEL_GENERIC && decode_mfma_supports(*p)) return launch_decode_mfma(*p, (hipStream_t)stream);
    // the packed table and computed cos/sin are read by the streaming kernel only
    if (p->packed_block_table || p->rope_freqs) return LAZYATTN_E_UNSUPPORTED;
    if (p->kernel != LAZYATTN_KERNEL_AUTO && p->kernel != LAZYATTN_KERNEL_GENERIC) return LAZYATTN_E_UNSUPPORTED;
    return launch_prefill_generic(*p, 1, (hipStream_t)stream);
}

extern "C" size_t lazyattn_paged_decode_workspace_bytes(const lazyattn_prefill_params *p) {
    if (!p || check_common(p, true) != LAZYATTN_OK) return 0;
    if (p->kernel == LAZYATTN_KERNEL_GENERIC || !decode_mfma_supports(*p)) return 0;
    return decode_workspace_bytes(*p);
}

extern "C" int lazyattn_rope_and_cache_write(const lazyattn_rope_write_params *p, void *stream) {
    if (!p) return LAZYATTN_E_NULL;
    const bool write = p->k_cache && p->slot_mapping;
    if ((p->rotate_q && !p->q) || ((p->rotate_k || write) && !p->k) || (write && (!p->v || !p->v_cache))) return LAZYATTN_E_NULL;
    if ((p->rotate_q || p->rotate_k) && (!p->positions || !p->cos_sin_cache)) return LAZYATTN_E_NULL;
    if (p->num_tokens < 0 || p->num_q_heads < 0 || p->num_kv_heads <= 0 || p->head_dim <= 0) return LAZYATTN_E_SHAPE;
    if (p->head_dim % 8 || p->rotary_dim % 16 || p->rotary_dim <= 0 || p->rotary_dim > p->head_dim) return LAZYATTN_E_SHAPE;
    if (p->dtype != LAZYATTN_F32 && p->dtype != LAZYATTN_BF16 && p->dtype != LAZYATTN_F16) return LAZYATTN_E_DTYPE;
    if (p->table_dtype != p->dtype && p->table_dtype != LAZYATTN_F32) return LAZYATTN_E_DTYPE;
    if (p->pos_bits != 32 && p->pos_bits != 64) return LAZYATTN_E_DTYPE;
    const int64_t vec = p->dtype == LAZYATTN_F32 ? 4 : 8;       // elements per 16 bytes
    if (p->q_stride[2] != 1 && p->q) return LAZYATTN_E_UNSUPPORTED;
    if (p->k_stride[2] != 1 || (write && p->v_stride[2] != 1)) return LAZYATTN_E_UNSUPPORTED;
    if ((p->q && (p->q_stride[0] % vec || p->q_stride[1] % vec || ((uintptr_t)p->q & 15))) ||
        p->k_stride[0] % vec || p->k_stride[1] % vec || ((uintptr_t)p->k & 15))
        return LAZYATTN_E_UNSUPPORTED;
    if ((p->rotate_q || p->rotate_k) &&
        (p->table_stride % (p->table_dtype == LAZYATTN_F32 ? 4 : 8) || ((uintptr_t)p->cos_sin_cache & 15)))
        return LAZYATTN_E_UNSUPPORTED;
    if (write) {
        const bool fp8 = p->cache_dtype == LAZYATTN_FP8_E4M3 || p->cache_dtype == LAZYATTN_FP8_E5M2;
        if (!fp8 && p->cache_dtype != p->dtype) return LAZYATTN_E_DTYPE;
        if (fp8 && (!p->k_scale || !p->v_scale)) return LAZYATTN_E_NULL;
        if (p->slot_bits != 32 && p->slot_bits != 64) return LAZYATTN_E_DTYPE;
        if (p->block_size <= 0 || p->x <= 0 || p->head_dim % p->x) return LAZYATTN_E_SHAPE;
        if (p->v_stride[0] % vec || p->v_stride[1] % vec || ((uintptr_t)p->v & 15)) return LAZYATTN_E_UNSUPPORTED;
        if (p->kc_stride[4] != 1) return LAZYATTN_E_UNSUPPORTED;
        // an fp8 K chunk is written as one 8-byte store: the innermost cache axis must hold whole chunks
        if (fp8 && p->x % 8) return LAZYATTN_E_UNSUPPORTED;
        // a K chunk of 8 elements is one store when x is a multiple of 8 (16-byte aligned for 2-byte types,
        // 8-byte aligned for fp8); x = 4 (fp32 caches) is written element-wise
        if (p->x % 8 == 0 &&
            (((uintptr_t)p->k_cache & 15) || p->kc_stride[0] % 16 || p->kc_stride[1] % 16 || p->kc_stride[2] % 8 || p->kc_stride[3] % 8))
            return LAZYATTN_E_UNSUPPORTED;
    }
    if (p->num_tokens == 0) return LAZYATTN_OK;
    return launch_rope_cache_write(*p, (hipStream_t)stream);
}

extern "C" int lazyattn_build_rotation_metadata(const int32_t *doc_lens, const int32_t *doc_lens_padded,
                                                const int32_t *doc_start, int32_t batch, int32_t block_size,
                                                int32_t zero_offsets, int32_t *q_offset, int32_t *q_mask,
                                                int64_t row_stride, int32_t row_len, int32_t *max_offset, void *stream) {
    if (!doc_lens || !doc_lens_padded || !doc_start || !q_offset || !q_mask) return LAZYATTN_E_NULL;
    if (batch < 0 || block_size <= 0 || row_len <= 0 || row_stride < row_len) return LAZYATTN_E_SHAPE;
    return launch_rotation_metadata(doc_lens, doc_lens_padded, doc_start, batch, block_size, zero_offsets, q_offset, q_mask,
                                    row_stride, row_len, max_offset, (hipStream_t)stream);
}

extern "C" int lazyattn_pack_block_table(const int32_t *block_table, int64_t bt_stride, const int32_t *q_offset,
                                         const int32_t *q_mask, int64_t row_stride, const int32_t *rows, int32_t n_rows,
                                         int32_t row_len, int64_t *packed, int64_t packed_stride, void *stream) {
    if (!block_table || !q_offset || !q_mask || !packed) return LAZYATTN_E_NULL;
    if (n_rows < 0 || row_len < 0 || bt_stride < row_len || row_stride < row_len || packed_stride < row_len) return LAZYATTN_E_SHAPE;
    return launch_pack_block_table(block_table, bt_stride, q_offset, q_mask, row_stride, rows, n_rows, row_len, packed,
                                   packed_stride, (hipStream_t)stream);
}

extern "C" int lazyattn_reposition_blocks(const lazyattn_reposition_params *p, void *stream) {
    if (!p || !p->k_cache || !p->v_cache || !p->items || !p->cos_sin_cache) return LAZYATTN_E_NULL;
    if (p->num_items < 0 || p->num_kv_heads <= 0 || p->head_dim <= 0 || p->head_dim % 16 || p->block_size <= 0 || p->x <= 0 ||
        p->head_dim % p->x)
        return LAZYATTN_E_SHAPE;
    if (p->dtype != LAZYATTN_F32 && p->dtype != LAZYATTN_BF16 && p->dtype != LAZYATTN_F16) return LAZYATTN_E_DTYPE;
    if (p->table_dtype != p->dtype && p->table_dtype != LAZYATTN_F32) return LAZYATTN_E_DTYPE;
    const int esz = p->dtype == LAZYATTN_F32 ? 4 : 2;
    // the V block is copied as one contiguous run of 16-byte pieces; K chunks of 8 are single accesses when x allows
    if (p->kc_stride[4] != 1 || p->vc_stride[3] != 1 || p->vc_stride[2] != p->block_size ||
        p->vc_stride[1] != (int64_t)p->head_dim * p->block_size)
        return LAZYATTN_E_UNSUPPORTED;
    if (((uintptr_t)p->k_cache & 15) || ((uintptr_t)p->v_cache & 15) || ((uintptr_t)p->cos_sin_cache & 15) ||
        (p->vc_stride[0] * esz) % 16 || ((int64_t)p->num_kv_heads * p->head_dim * p->block_size * esz) % 16 ||
        (p->table_stride * (p->table_dtype == LAZYATTN_F32 ? 4 : 2)) % 16)
        return LAZYATTN_E_UNSUPPORTED;
    if (p->x % 8 == 0 && ((p->kc_stride[0] * esz) % 16 || (p->kc_stride[1] * esz) % 16 || (p->kc_stride[2] * esz) % 16 ||
                          (p->kc_stride[3] * esz) % 16))
        return LAZYATTN_E_UNSUPPORTED;
    if (p->num_items == 0) return LAZYATTN_OK;
    return launch_block_reposition(*p, (hipStream_t)stream);
}

extern "C" int lazyattn_build_cos_sin_cache(void *out, int32_t out_dtype, int64_t row_stride,
                                            int32_t max_position, int32_t rotary_dim, double base,
                                            int32_t rope_type, double scaling_factor,
                                            double low_freq_factor, double high_freq_factor,
                                            int32_t orig_max_position, void *stream) {
    if (!out) return LAZYATTN_E_NULL;
    if (max_position < 0 || rotary_dim <= 0 || rotary_dim % 2 || row_stride < rotary_dim)
        return LAZYATTN_E_SHAPE;
    if (rope_type != 0 && rope_type != 1) return LAZYATTN_E_UNSUPPORTED;
    if (rope_type == 1 && (high_freq_factor == low_freq_factor || scaling_factor == 0.0))
        return LAZYATTN_E_SHAPE;
    return launch_cos_sin_table(out, out_dtype, row_stride, max_position, rotary_dim, base, rope_type,
                                scaling_factor, low_freq_factor, high_freq_factor, orig_max_position,
                                (hipStream_t)stream);
}

extern "C" int lazyattn_pack_cos_sin_cache(const void *table, void *packed, int32_t dtype, int64_t row_stride,
                                           int32_t rows, int32_t rotary_dim, void *stream) {
    if (!table || !packed) return LAZYATTN_E_NULL;
    if (rows < 0 || rotary_dim <= 0 || rotary_dim % 16 || row_stride < rotary_dim) return LAZYATTN_E_SHAPE;
    return launch_pack_cos_sin(table, packed, dtype, row_stride, rows, rotary_dim, (hipStream_t)stream);
}

extern "C" const char *lazyattn_error_string(int code) {
    switch (code) {
        case LAZYATTN_OK: return "ok";
        case LAZYATTN_E_NULL: return "a required pointer is null";
        case LAZYATTN_E_SHAPE: return "inconsistent sizes";
        case LAZYATTN_E_DTYPE: return "unsupported element type combination";
        case LAZYATTN_E_UNSUPPORTED: return "request not supported by the selected kernel";
        case LAZYATTN_E_WORKSPACE: return "workspace missing or too small";
        case LAZYATTN_E_LAUNCH: return "kernel launch failed";
        case LAZYATTN_E_SCRATCH_LIMIT: return "the call needs more split-KV scratch than the library's static buffer holds";
        default: return "unknown error";
    }
}

extern "C" int lazyattn_abi_version(void) { return 3; }
