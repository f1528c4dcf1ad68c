// Per-page rotation metadata of a batch, produced on the device.
//
// Same integers as metadata_for_lazy_attention / metadata_for_mepic
// (lazy_attn/lazy/core/sched/scheduler.py:758-787) written straight into the [batch, row_len]
// device buffers the attention kernels read (the reference fills host rows request by request
// and copies two [num_reqs, max_blocks] arrays to the device every step,
// worker/gpu_model_runner.py:193-239):
//   every page of document d:  q_offset = (total padding + true lengths of the documents before d) + 1
//   last page of document d:   q_mask   = padded_len[d] - true_len[d]
//   the page after the last document (the query's): q_offset = 1
//   everything else 0; with zero_offsets (un-rotated-cache variant) all q_offset are 0.
// One workgroup per request; documents are given in CSR form (doc_start[b] .. doc_start[b+1]).
#include "common.hpp"

namespace lazyattn {

__global__ void __launch_bounds__(256)
rotation_metadata_kernel(const int32_t *doc_lens, const int32_t *doc_lens_padded, const int32_t *doc_start,
                         int block_size, int zero_offsets, int32_t *q_offset, int32_t *q_mask, int64_t row_stride,
                         int row_len, int32_t *max_offset) {
    const int b = blockIdx.x, tid = threadIdx.x;
    const int d0 = doc_start[b], d1 = doc_start[b + 1];
    int32_t *qo = q_offset + b * row_stride, *qm = q_mask + b * row_stride;
    for (int j = tid; j < row_len; j += blockDim.x) { qo[j] = 0; qm[j] = 0; }
    __shared__ int s_padding;
    if (tid == 0) {
        int pad = 0;
        for (int d = d0; d < d1; ++d) pad += doc_lens_padded[d] - doc_lens[d];
        s_padding = pad;
    }
    __syncthreads();
    // each thread walks the documents before its own: requests hold tens of documents, not thousands
    int query_page = 0, last_offset = 0;
    for (int d = d0 + tid; d < d1; d += blockDim.x) {
        int shift = s_padding, page = 0;
        for (int e = d0; e < d; ++e) { shift += doc_lens[e]; page += doc_lens_padded[e] / block_size; }
        const int pages = doc_lens_padded[d] / block_size;
        for (int j = page; j < page + pages && j < row_len; ++j) qo[j] = zero_offsets ? 0 : shift + 1;
        if (pages > 0 && page + pages - 1 < row_len) qm[page + pages - 1] = doc_lens_padded[d] - doc_lens[d];
        if (d == d1 - 1) { query_page = page + pages; last_offset = shift + 1; }
    }
    // the thread that owns the last document also writes the query page and the request's largest offset
    const int owner = d1 > d0 ? (d1 - 1 - d0) % blockDim.x : 0;
    if (tid == owner) {
        if (query_page < row_len) qo[query_page] = zero_offsets ? 0 : 1;
        if (max_offset) max_offset[b] = d1 > d0 ? last_offset : 0;
    }
}

// packed[r, j] = block_table[r, j] << 32 | q_offset[r, j] << 16 | q_mask[r, j] for the listed rows
// (rows == nullptr: rows 0 .. n_rows-1): the table the block-uniform decode kernels of the
// reference read (worker/gpu_model_runner.py:296-340, five tensor ops per row there).
__global__ void __launch_bounds__(256)
pack_block_table_kernel(const int32_t *block_table, int64_t bt_stride, const int32_t *q_offset, const int32_t *q_mask,
                        int64_t row_stride, const int32_t *rows, int row_len, int64_t *packed, int64_t packed_stride) {
    const int r = rows ? rows[blockIdx.y] : (int)blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= row_len) return;
    const uint64_t blk = (uint32_t)block_table[r * bt_stride + j];
    const uint64_t off = (uint32_t)q_offset[r * row_stride + j] & 0xffffu;
    const uint64_t msk = (uint32_t)q_mask[r * row_stride + j] & 0xffffu;
    packed[r * packed_stride + j] = (int64_t)((blk << 32) | (off << 16) | msk);
}

int launch_pack_block_table(const int32_t *block_table, int64_t bt_stride, const int32_t *q_offset, const int32_t *q_mask,
                            int64_t row_stride, const int32_t *rows, int n_rows, int row_len, int64_t *packed,
                            int64_t packed_stride, hipStream_t stream) {
    if (n_rows <= 0 || row_len <= 0) return LAZYATTN_OK;
    hipLaunchKernelGGL(pack_block_table_kernel, dim3((row_len + 255) / 256, n_rows), dim3(256), 0, stream, block_table, bt_stride,
                       q_offset, q_mask, row_stride, rows, row_len, packed, packed_stride);
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

int launch_rotation_metadata(const int32_t *doc_lens, const int32_t *doc_lens_padded, const int32_t *doc_start, int batch,
                             int block_size, int zero_offsets, int32_t *q_offset, int32_t *q_mask, int64_t row_stride,
                             int row_len, int32_t *max_offset, hipStream_t stream) {
    if (batch <= 0) return LAZYATTN_OK;
    hipLaunchKernelGGL(rotation_metadata_kernel, dim3(batch), dim3(256), 0, stream, doc_lens, doc_lens_padded, doc_start,
                       block_size, zero_offsets, q_offset, q_mask, row_stride, row_len, max_offset);
    return hipGetLastError() == hipSuccess ? LAZYATTN_OK : LAZYATTN_E_LAUNCH;
}

}  // namespace lazyattn
