// Row copies between two jagged (or dense-per-batch) 2-D tensors and their per-batch concatenation: the data
// format either side of the attention path (cache (+) delta -> full K/V, full -> cache | delta).  Pure byte
// movement, bound by HBM bandwidth; results are bit-identical to an index copy by definition.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hstu {

struct JaggedCopyParams {
    char* left;
    char* right;
    char* joined;
    int64_t left_rs, right_rs, joined_rs;  // row strides in bytes
    int64_t row_bytes;
    const void* offsets_left;   // NULL = dense: exactly max_len_left rows per batch
    const void* offsets_right;
    int offsets_left_i64, offsets_right_i64;
    int batch;
    int max_len_left, max_len_right;
};

__device__ __forceinline__ int64_t jagged_offset(const void* offsets, int is_i64, int dense_len, int b) {
    if (!offsets) return (int64_t)dense_len * b;
    return is_i64 ? ((const int64_t*)offsets)[b] : (int64_t)((const int*)offsets)[b];
}

// One workgroup per (batch, block of ROWS joined rows).  joined row r of batch b is left row r if r < len_left(b),
// else right row r - len_left(b); the joined tensor starts batch b at offset_left[b] + offset_right[b].
// SPLIT = false: left, right -> joined (concat_2D_jagged); SPLIT = true: joined -> left, right (split_2D_jagged).
// VEC = bytes moved per thread and access (16, 8, 4, 2 or 1: the largest that divides row_bytes, every stride
// and every base address).
template <bool SPLIT, int VEC, int ROWS>
__global__ __launch_bounds__(256) void hstu_jagged_copy_kernel(const JaggedCopyParams p) {
    typedef __attribute__((ext_vector_type(4))) int v16;
    const int b = blockIdx.y;
    const int64_t ol = jagged_offset(p.offsets_left, p.offsets_left_i64, p.max_len_left, b);
    const int64_t orr = jagged_offset(p.offsets_right, p.offsets_right_i64, p.max_len_right, b);
    int64_t len_l = jagged_offset(p.offsets_left, p.offsets_left_i64, p.max_len_left, b + 1) - ol;
    int64_t len_r = jagged_offset(p.offsets_right, p.offsets_right_i64, p.max_len_right, b + 1) - orr;
    const int64_t r0 = (int64_t)blockIdx.x * ROWS;
    if (r0 >= len_l + len_r) return;
    const int64_t r1 = r0 + ROWS < len_l + len_r ? r0 + ROWS : len_l + len_r;
    const int64_t vec_per_row = p.row_bytes / VEC;
    const int64_t total = (r1 - r0) * vec_per_row;
    // four independent accesses per thread and round, loads first: a cold copy needs many bytes in flight
    for (int64_t i0 = threadIdx.x; i0 < total; i0 += 1024) {
        char* src[4];
        char* dst[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t i = i0 + j * 256;
            const int64_t ii = i < total ? i : i0;  // lanes past the end repeat their first access
            const int64_t r = r0 + ii / vec_per_row;
            const int64_t c = (ii % vec_per_row) * VEC;
            char* part = r < len_l ? p.left + (ol + r) * p.left_rs : p.right + (orr + r - len_l) * p.right_rs;
            char* whole = p.joined + (ol + orr + r) * p.joined_rs;
            src[j] = (SPLIT ? whole : part) + c;
            dst[j] = (SPLIT ? part : whole) + c;
        }
        if (VEC == 16) {
            v16 x[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) x[j] = *(const v16*)src[j];
#pragma unroll
            for (int j = 0; j < 4; ++j) *(v16*)dst[j] = x[j];
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (VEC == 8) *(int64_t*)dst[j] = *(const int64_t*)src[j];
                else if (VEC == 4) *(int*)dst[j] = *(const int*)src[j];
                else if (VEC == 2) *(short*)dst[j] = *(const short*)src[j];
                else *dst[j] = *src[j];
            }
        }
    }
}

// joined[offsets_joined[b+1] - tail_len + i] = tail[b * tail_len + i]: writes a dense block of `tail_len` rows per
// batch over the last rows of every sequence of a jagged tensor, in place.  With a K/V cache kept in the layout
// "history rows, then tail_len spare rows" per sequence this replaces the concatenation of the whole history with
// the new rows by a copy of the new rows alone.  One workgroup per (batch, block of ROWS tail rows).
template <int VEC, int ROWS>
__global__ __launch_bounds__(256) void hstu_jagged_write_tail_kernel(char* joined, int64_t joined_rs, const void* offsets,
                                                                     int offsets_i64, const char* tail, int64_t tail_rs,
                                                                     int64_t row_bytes, int tail_len) {
    typedef __attribute__((ext_vector_type(4))) int v16;
    const int b = blockIdx.y;
    const int64_t end = jagged_offset(offsets, offsets_i64, 0, b + 1);
    const int64_t start = jagged_offset(offsets, offsets_i64, 0, b);
    if (end - start < tail_len) return;  // contract: every sequence holds at least tail_len rows
    const int r0 = blockIdx.x * ROWS;
    if (r0 >= tail_len) return;
    const int r1 = r0 + ROWS < tail_len ? r0 + ROWS : tail_len;
    const int64_t vec_per_row = row_bytes / VEC;
    const int64_t total = (int64_t)(r1 - r0) * vec_per_row;
    for (int64_t i = threadIdx.x; i < total; i += 256) {
        const int64_t r = r0 + i / vec_per_row;
        const int64_t c = (i % vec_per_row) * VEC;
        const char* src = tail + ((int64_t)b * tail_len + r) * tail_rs + c;
        char* dst = joined + (end - tail_len + r) * joined_rs + c;
        if (VEC == 16) *(v16*)dst = *(const v16*)src;
        else if (VEC == 8) *(int64_t*)dst = *(const int64_t*)src;
        else if (VEC == 4) *(int*)dst = *(const int*)src;
        else if (VEC == 2) *(short*)dst = *(const short*)src;
        else *dst = *src;
    }
}

}  // namespace hstu
