/*
 * hstu_uqvk.h -- C ABI of libhstu_uqvk.so: the producer of q, k, v for the HSTU attention path on gfx950.
 *
 * Replaces `hstu_compute_uqvk` (generative_recommenders/ops/hstu_compute.py:54-104):
 *     normed = layer_norm(x, weight, bias, eps)                 (fp32 statistics, result in x's type,
 *                                                                ops/pytorch/pt_layer_norm.py:24-39)
 *     uvqk   = uvqk_bias + normed @ uvqk_weight                 [L, (2*hidden + 2*attn) * H]
 *     u, v, q, k = split(uvqk, [hidden*H, hidden*H, attn*H, attn*H]);  u = silu(u)
 * All four results stay column slices of ONE [L, n_out] buffer -- the layout the attention entry points read in
 * place through their row / head strides -- so nothing is copied on the way to `hstu_hip_mha_fwd`.
 *
 * The layer norm is a hand-written kernel (one wave per row, HBM-bound).  The matrix product is a plain GEMM and
 * goes to hipBLASLt, with the bias and, for the u columns, the SiLU in the GEMM's epilogue.  This library is
 * separate from libhstu_hip.so so that the attention library does not depend on hipBLASLt.
 * Plain pointers and sizes; device pointers on the current HIP device; asynchronous on the stream given.
 */
#ifndef HSTU_UQVK_H_
#define HSTU_UQVK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes: 0 ok; negative values as in hstu_hip.h (-1 NULL pointer, -2 dtype, -4 alignment, -5 shape,
 * -6 unsupported, -7 HIP launch failure), -9 hipBLASLt failure (see hstu_uqvk_last_error()). */
enum { HSTU_UQVK_ERR_BLASLT = -9 };

typedef struct HstuUqvkArgs {
    const void* x;             /* [rows, d_model], bf16 or fp16, innermost stride 1 */
    int64_t x_row_stride;      /* elements */
    const void* norm_weight;   /* [d_model], same type */
    const void* norm_bias;     /* [d_model] */
    float norm_eps;
    const void* uvqk_weight;   /* [d_model, n_out] row-major, dense */
    const void* uvqk_bias;     /* [n_out] */
    void* uvqk;                /* [rows, n_out] dense output: u | v | q | k column blocks, u already through SiLU */
    int64_t rows;
    int32_t d_model;           /* multiple of 8, at most 4096 */
    int32_t heads, attn_dim, hidden_dim;  /* n_out = (2 * hidden_dim + 2 * attn_dim) * heads */
    int32_t dtype;             /* 0 = bf16, 1 = fp16 (HstuDtype of hstu_hip.h) */
    void* workspace;           /* hstu_uqvk_workspace_bytes() bytes, 256-byte aligned: the normalised x and the
                                  GEMM's scratch */
    int64_t workspace_bytes;
} HstuUqvkArgs;

size_t hstu_uqvk_workspace_bytes(const HstuUqvkArgs* args);

/* layer norm + GEMM + bias + split + SiLU(u), as described at the top. */
int hstu_uqvk_forward(const HstuUqvkArgs* args, void* stream);

/* Only the layer norm: out[r] = (x[r] - mean) * rsqrt(var + eps) * weight + bias, statistics in fp32
 * (ops/pytorch/pt_layer_norm.py:24-39).  Strides in elements. */
int hstu_uqvk_layer_norm(const void* x, int64_t x_row_stride, const void* weight, const void* bias, float eps, void* out,
                         int64_t out_row_stride, int64_t rows, int32_t d_model, int32_t dtype, void* stream);

const char* hstu_uqvk_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_UQVK_H_ */
