/*
 * hstu_linear.h -- C ABI of libhstu_linear.so: the producer of q, k, v for the HSTU attention path on gfx950 and the
 * consumer of its output.
 *
 * Producer: replaces `hstu_compute_uqvk` (generative_recommenders/ops/hstu_compute.py:54-104):
 *     normed = layer_norm(x, weight, bias, eps)                 (fp32 statistics, result in x's type,
 *                                                                ops/pytorch/pt_layer_norm.py:24-39)
 *     uvqk   = uvqk_bias + normed @ uvqk_weight                 [L, (2*hidden + 2*attn) * H]
 *     u, v, q, k = split(uvqk, [hidden*H, hidden*H, attn*H, attn*H]);  u = silu(u)
 * All four results stay column slices of ONE [L, n_out] buffer -- the layout the attention entry points read in
 * place through their row / head strides -- so nothing is copied on the way to `hstu_hip_mha_fwd`.
 *
 * Two paths.  Fused (the usual shapes, see `path`): one hand-written kernel that keeps a wave's 32 normalised rows in
 * registers as MFMA operands, streams the weight through LDS and applies bias and SiLU before the store -- x is read
 * once, uvqk written once, nothing else touches HBM.  Library path (any shape): a layer-norm kernel (one wave per row)
 * and hipBLASLt with the bias and, for the u columns, the SiLU in the GEMM's epilogue.  This library is separate from
 * libhstu_hip.so so that the attention library does not depend on hipBLASLt.
 * Plain pointers and sizes; device pointers on the current HIP device; asynchronous on the stream given.
 */
#ifndef HSTU_LINEAR_H_
#define HSTU_LINEAR_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes: 0 ok; negative values as in hstu_hip.h (-1 NULL pointer, -2 dtype, -4 alignment, -5 shape,
 * -6 unsupported, -7 HIP launch failure), -9 hipBLASLt failure (see hstu_linear_last_error()). */
enum { HSTU_LINEAR_ERR_BLASLT = -9 };

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
                                  GEMM's scratch (unused by the fused kernel; may then be NULL) */
    int64_t workspace_bytes;
    int32_t path;              /* 0 = automatic: the fused kernel (layer norm, product, bias, SiLU in one pass, the
                                  normalised rows held in registers) when d_model is 128, 256, 384 or 512 and
                                  hidden_dim * heads and n_out are multiples of 128, else the library path;
                                  1 = library path (layer-norm kernel + hipBLASLt); 2 = fused kernel or status -6;
                                  3 = layer-norm kernel + the hand-written GEMM kernel of the output projection with the
                                  bias as the start of the sums and SiLU(u) in its epilogue (d_model a multiple of 64,
                                  hidden_dim * heads and n_out multiples of 256, else status -6): never the automatic
                                  choice, it is the slowest of the three at the widths measured */
    /* Optional e4m3 hand-off to the fp8 attention path (the counterpart of the reference's fp8 producer,
     * ops/cpp/cuda_hstu_preprocess_and_attention.py:262-282): the fused kernel writes the v | q | k column blocks a second
     * time as e4m3 bytes, qkv_fp8[r, c] = e4m3(float(uvqk[r, hidden*H + c]) * (1.0f / scale)) with the scale of the block
     * c falls in (round to nearest even, clamped to +-448; `uvqk` holds the values already rounded to its 16-bit type),
     * and raises qkv_absmax[0..2] to max |uvqk| over this call's rows of v, q, k (bit patterns of non-negative floats,
     * atomicMax; the caller zeroes them): the per-tensor scales of the NEXT batch, e.g. absmax / 448.  NULL = off.
     * Needs the fused kernel (path 0 or 2 with a shape it takes), else status -6. */
    void* qkv_fp8;             /* [rows, (hidden_dim + 2 * attn_dim) * heads] dense, 16-byte aligned */
    float v_scale, q_scale, k_scale;  /* > 0 */
    void* qkv_absmax;          /* 3 floats of device memory */
} HstuUqvkArgs;

size_t hstu_uqvk_workspace_bytes(const HstuUqvkArgs* args);

/* layer norm + GEMM + bias + split + SiLU(u), as described at the top. */
int hstu_uqvk_forward(const HstuUqvkArgs* args, void* stream);

/* Only the layer norm: out[r] = (x[r] - mean) * rsqrt(var + eps) * weight + bias, statistics in fp32
 * (ops/pytorch/pt_layer_norm.py:24-39).  Strides in elements. */
int hstu_uqvk_layer_norm(const void* x, int64_t x_row_stride, const void* weight, const void* bias, float eps, void* out,
                         int64_t out_row_stride, int64_t rows, int32_t d_model, int32_t dtype, void* stream);

/*
 * Consumer: replaces `hstu_compute_output` (generative_recommenders/ops/hstu_compute.py:107-214) in its forward
 * form, i.e. `pytorch_hstu_compute_output` (ops/pytorch/pt_hstu_linear.py:88-124); dropout: see `dropout_ratio`:
 *     y   = norm_mul(attn, u)                      (pt_hstu_linear.py:24-85, statistics and product in fp32)
 *              layer norm : y = act(u) * layer_norm(attn) over the whole row, act in {none, sigmoid, silu};
 *                           joined = [u] | [attn] | y, a block present when concat_u / concat_x is set
 *              group norm : y = u * group_norm(attn) per head of linear_dim columns, one weight and bias per head;
 *                           joined = u | attn | y only when concat_u AND concat_x, else y alone (as the reference)
 *              silu_u     : layer norm: the copied u block goes through SiLU; group norm: u does before both uses
 *     out = x + joined @ output_weight             [rows, d_out]
 * Two paths (see `path`).  Library path (any shape): the norm / multiply / concatenate step is one hand-written kernel
 * (one wave per row, HBM-bound) that writes `joined` in the inputs' type; the product with the residual as the GEMM's
 * C operand runs on hipBLASLt.  Concatenating path (d_out a multiple of 256): the same norm-multiply kernel writes y alone (and
 * SiLU(u) where that is a block of `joined`), and a hand-written GEMM kernel reads the blocks of `joined` where they
 * are -- u and attn in the caller's tensors, y in the workspace -- so that `joined` is never written: 1.15 ms against
 * the library path's 1.39 ms at the benchmark's shape (524288 rows, 3 x 512 -> 512).
 */
enum { HSTU_MUL_U_NONE = 0, HSTU_MUL_U_SIGMOID = 1, HSTU_MUL_U_SILU = 2 };

typedef struct HstuOutputArgs {
    const void* attn;          /* [rows, heads * linear_dim], bf16 or fp16, innermost stride 1 */
    int64_t attn_row_stride;   /* elements */
    const void* u;             /* [rows, heads * linear_dim] */
    int64_t u_row_stride;
    const void* x;             /* [rows, d_out]: the residual */
    int64_t x_row_stride;
    const void* norm_weight;   /* layer norm: [heads * linear_dim]; group norm: [heads] */
    const void* norm_bias;
    float norm_eps;
    const void* output_weight; /* [blocks * heads * linear_dim, d_out] row-major, dense; blocks = 1 + copied blocks */
    void* out;                 /* [rows, d_out] dense */
    int64_t rows;
    int32_t d_out;             /* multiple of 8 */
    int32_t heads, linear_dim; /* heads * linear_dim: multiple of 8, at most 4096; group norm: linear_dim / 8 a power of two <= 64 */
    int32_t concat_u, concat_x, group_norm, silu_u;  /* 0 / 1 */
    int32_t mul_u_activation;  /* HSTU_MUL_U_*; layer norm only */
    int32_t dtype;             /* 0 = bf16, 1 = fp16 */
    void* workspace;           /* hstu_output_workspace_bytes() bytes, 256-byte aligned: library path: `joined` and the
                                  GEMM's scratch; concatenating path: y (and SiLU(u)) */
    int64_t workspace_bytes;
    int32_t path;              /* 1 = library path (norm-mul kernel + hipBLASLt); 2 = concatenating path (norm-mul kernel
                                  + hand-written GEMM over the blocks where they are): needs d_out a multiple of 256 and heads *
                                  linear_dim a multiple of 64 (and, with group norm, no SiLU on a copied u), else status
                                  -6; 0 = the concatenating path where it applies and rows >= 32768, else the library */
    /* Dropout of `joined` (`F.dropout(y, p, training)` at the end of pytorch_norm_mul_dropout, pt_hstu_linear.py:80-84): the
     * whole concatenation goes through it, in fp32, before it is rounded; survivors are multiplied by 1 / (1 - ratio).
     * Element (r, c) of the [rows, blocks * heads * linear_dim] matrix is kept when word c % 4 of
     * Philox4x32-10(counter = {(r * width + c) / 4, dropout_offset}, key = dropout_seed) is >= floor(ratio * 2^32): a pure
     * function of (seed, offset, r, c), so hstu_output_dropout_mask returns the mask of any earlier call.  0 = no
     * dropout (inference, `training=False`); with a ratio > 0 path 2 is refused (-6) and path 0 takes the library path. */
    float dropout_ratio;       /* [0, 1) */
    uint64_t dropout_seed, dropout_offset;
} HstuOutputArgs;

size_t hstu_output_workspace_bytes(const HstuOutputArgs* args);

/* norm_mul + concatenation + GEMM + residual, as described above. */
int hstu_output_forward(const HstuOutputArgs* args, void* stream);

/* Only the first step (`pytorch_norm_mul_dropout`, pt_hstu_linear.py:24-85): writes `joined`
 * [rows, blocks * heads * linear_dim] with row stride `joined_row_stride` elements.  Reads attn, u, norm_weight,
 * norm_bias, norm_eps, rows, heads, linear_dim, the five flags, dtype and the dropout fields of `args`; the other fields are
 * ignored. */
int hstu_output_norm_mul(const HstuOutputArgs* args, void* joined, int64_t joined_row_stride, void* stream);

/* keep[r * width + c] (one byte per element, 1 = kept) for the mask a call with the same ratio, seed and offset applied to a
 * `joined` of `width` columns (a multiple of 8): what the backward of the dropout multiplies by, times 1 / (1 - ratio).
 * `keep`: rows * width bytes of device memory, 4-byte aligned. */
int hstu_output_dropout_mask(float ratio, uint64_t seed, uint64_t offset, int64_t rows, int64_t width, void* keep, void* stream);

const char* hstu_linear_last_error(void);

/* Library version, major*10000 + minor*100 + patch.  101: HstuUqvkArgs gained qkv_fp8 / v_scale / q_scale / k_scale /
 * qkv_absmax and HstuOutputArgs gained dropout_ratio / dropout_seed / dropout_offset, all at the end of the structs: a
 * caller built against an older header passes shorter structs and must be rebuilt. */
int hstu_linear_version(void);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_LINEAR_H_ */
