// C ABI of libhstu_linear.so: layer norm and norm-multiply-concatenate kernels, hipBLASLt GEMMs with fused bias /
// SiLU epilogues and the residual as C operand, the fused q/k/v producer and the concatenating output GEMM.
// Declarations and the reference interfaces they replace are in include/hstu_linear.h.
#include "hstu_linear.h"

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>

#include "hstu_philox.h"
#include "hstu_uqvk_kernel.h"
#include "hstu_output_kernel.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;

thread_local char g_last_error[256] = "";

// Sum over the 64 lanes of a wave, result in every lane.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
    return v;
}

// One wave per row, rows dealt to the waves of the grid with a stride.  A lane holds NCH chunks of 8 elements
// (chunk c of the row goes to lane c % 64), loaded once; mean and variance in fp32 (two passes over the
// registers, as torch's layer_norm does), weight and bias loaded once per wave.
template <class V8, int NCH>
__global__ __launch_bounds__(256) void hstu_layer_norm_kernel(const char* x, int64_t x_rs, const char* weight, const char* bias,
                                                              float eps, char* out, int64_t out_rs, int64_t rows, int d) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    const int chunks = d >> 3;
    float w[NCH][8], b[NCH][8];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = lane + 64 * i;
        if (c < chunks) {
            const V8 wv = *(const V8*)(weight + (int64_t)c * 16), bv = *(const V8*)(bias + (int64_t)c * 16);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                w[i][j] = (float)wv[j];
                b[i][j] = (float)bv[j];
            }
        }
    }
    const float inv_d = 1.0f / (float)d;
    for (int64_t r = wave; r < rows; r += nwaves) {
        float v[NCH][8];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = lane + 64 * i;
            if (c < chunks) {
                const V8 xv = *(const V8*)(x + (r * x_rs + (int64_t)c * 8) * 2);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    v[i][j] = (float)xv[j];
                    sum += v[i][j];
                }
            }
        }
        const float mean = wave_sum(sum) * inv_d;
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < NCH; ++i)
            if (lane + 64 * i < chunks)
#pragma unroll
                for (int j = 0; j < 8; ++j) sq += (v[i][j] - mean) * (v[i][j] - mean);
        const float rstd = __builtin_amdgcn_rsqf(wave_sum(sq) * inv_d + eps);
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = lane + 64 * i;
            if (c < chunks) {
                V8 o;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = (decltype(o[0] + o[0]))((v[i][j] - mean) * rstd * w[i][j] + b[i][j]);
                *(V8*)(out + (r * out_rs + (int64_t)c * 8) * 2) = o;
            }
        }
    }
}

int launch_layer_norm(const void* x, int64_t x_rs, const void* weight, const void* bias, float eps, void* out, int64_t out_rs,
                      int64_t rows, int d, int dtype, hipStream_t stream) {
    if (rows < 0 || d <= 0 || (d & 7) != 0 || d > 4096 || x_rs < d || out_rs < d || (x_rs & 7) != 0 || (out_rs & 7) != 0) return -5;
    if (dtype != 0 && dtype != 1) return -2;
    if (rows == 0) return 0;
    if (!x || !weight || !bias || !out) return -1;
    if ((((uintptr_t)x | (uintptr_t)weight | (uintptr_t)bias | (uintptr_t)out) & 15) != 0) return -4;
    long long blocks = (rows + 3) / 4;
    if (blocks > 256 * 16) blocks = 256 * 16;  // 16 four-wave workgroups per CU keep the loads in flight
    const int nch = (d / 8 + 63) / 64;
#define HSTU_LN(V8, N)                                                                                                          \
    hipLaunchKernelGGL((hstu_layer_norm_kernel<V8, N>), dim3((unsigned)blocks), dim3(256), 0, stream, (const char*)x, x_rs,         \
                       (const char*)weight, (const char*)bias, eps, (char*)out, out_rs, rows, d)
    if (dtype == 0) {
        if (nch <= 1) HSTU_LN(bf16x8_t, 1); else if (nch <= 2) HSTU_LN(bf16x8_t, 2); else if (nch <= 4) HSTU_LN(bf16x8_t, 4); else HSTU_LN(bf16x8_t, 8);
    } else {
        if (nch <= 1) HSTU_LN(f16x8_t, 1); else if (nch <= 2) HSTU_LN(f16x8_t, 2); else if (nch <= 4) HSTU_LN(f16x8_t, 4); else HSTU_LN(f16x8_t, 8);
    }
#undef HSTU_LN
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(g_last_error, sizeof(g_last_error), "layer norm kernel launch: %s", hipGetErrorString(e));
        return -7;
    }
    return 0;
}

// ---- norm * u, concatenated with the copied blocks ------------------------------------------------------------------
struct NormMulParams {
    const char *attn, *u, *weight, *bias;
    char* joined;
    int64_t attn_rs, u_rs, joined_rs, rows;  // strides in elements
    float eps;
    int d, group_lanes;                      // row width; lanes per head (group norm)
    int off_u, off_x, off_y;                 // column offsets of the blocks in `joined`, -1 = block absent
    int silu_u, mul_act;
    hstu::DropoutParams drop;                // thresh 0: no dropout
    int64_t width;                           // logical width of `joined` (all blocks): the mask's row pitch
};

// Eight consecutive elements starting at column `col` (a multiple of 8) of row r: dropped or scaled, in fp32.
template <class V8, class E>
__device__ __forceinline__ V8 dropout8(const hstu::DropoutParams& d, int64_t r, int64_t width, int64_t col, const float (&x)[8]) {
    const uint64_t group = (uint64_t)(r * width + col) >> 2;
    const hstu::PhiloxWords a = hstu::dropout_words(d, group), b = hstu::dropout_words(d, group + 1);
    V8 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        out[j] = (E)(a.w[j] >= d.thresh ? x[j] * d.scale : 0.f);
        out[4 + j] = (E)(b.w[j] >= d.thresh ? x[4 + j] * d.scale : 0.f);
    }
    return out;
}

// keep[r * width + c] = 1 where the element survives: what the backward pass multiplies by (times the scale).
__global__ __launch_bounds__(256) void hstu_dropout_mask_kernel(hstu::DropoutParams d, int64_t groups, unsigned char* keep) {
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        const hstu::PhiloxWords a = hstu::dropout_words(d, (uint64_t)g);
        uchar4 k;
        k.x = a.w[0] >= d.thresh, k.y = a.w[1] >= d.thresh, k.z = a.w[2] >= d.thresh, k.w = a.w[3] >= d.thresh;
        ((uchar4*)keep)[g] = k;
    }
}

__device__ __forceinline__ float sigmoid_f(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// One wave per row as in the layer norm kernel.  GROUP: statistics per head (aligned groups of `group_lanes` lanes hold
// one head's chunks, so the sums run over xor distances below group_lanes) and one weight / bias per head.
template <class V8, int NCH, bool GROUP>
__global__ __launch_bounds__(256) void hstu_norm_mul_kernel(NormMulParams p) {
    typedef decltype(V8{}[0] + V8{}[0]) E;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    const int chunks = p.d >> 3;
    float w[NCH][GROUP ? 1 : 8], b[NCH][GROUP ? 1 : 8];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = lane + 64 * i;
        if (c < chunks) {
            if constexpr (GROUP) {
                const int head = c / p.group_lanes;
                w[i][0] = (float)((const E*)p.weight)[head];
                b[i][0] = (float)((const E*)p.bias)[head];
            } else {
                const V8 wv = *(const V8*)(p.weight + (int64_t)c * 16), bv = *(const V8*)(p.bias + (int64_t)c * 16);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    w[i][j] = (float)wv[j];
                    b[i][j] = (float)bv[j];
                }
            }
        }
    }
    const float inv_n = GROUP ? 1.0f / (float)(p.group_lanes * 8) : 1.0f / (float)p.d;
    for (int64_t r = wave; r < p.rows; r += nwaves) {
        float v[NCH][8];
        V8 uraw[NCH], xraw[NCH];
        float sum[NCH];
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = lane + 64 * i;
            sum[i] = 0.f;
            if (c < chunks) {
                xraw[i] = *(const V8*)(p.attn + (r * p.attn_rs + (int64_t)c * 8) * 2);
                uraw[i] = *(const V8*)(p.u + (r * p.u_rs + (int64_t)c * 8) * 2);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    v[i][j] = (float)xraw[i][j];
                    sum[i] += v[i][j];
                }
            }
        }
        float mean[NCH], rstd[NCH];
        if constexpr (GROUP) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                for (int d = 1; d < p.group_lanes; d <<= 1) sum[i] += __shfl_xor(sum[i], d, 64);
                mean[i] = sum[i] * inv_n;
            }
        } else {
            float t = 0.f;
#pragma unroll
            for (int i = 0; i < NCH; ++i) t += sum[i];
            t = wave_sum(t) * inv_n;
#pragma unroll
            for (int i = 0; i < NCH; ++i) mean[i] = t;
        }
        float sq[NCH];
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            sq[i] = 0.f;
            if (lane + 64 * i < chunks)
#pragma unroll
                for (int j = 0; j < 8; ++j) sq[i] += (v[i][j] - mean[i]) * (v[i][j] - mean[i]);
        }
        if constexpr (GROUP) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                for (int d = 1; d < p.group_lanes; d <<= 1) sq[i] += __shfl_xor(sq[i], d, 64);
                rstd[i] = __builtin_amdgcn_rsqf(sq[i] * inv_n + p.eps);
            }
        } else {
            float t = 0.f;
#pragma unroll
            for (int i = 0; i < NCH; ++i) t += sq[i];
            t = __builtin_amdgcn_rsqf(wave_sum(t) * inv_n + p.eps);
#pragma unroll
            for (int i = 0; i < NCH; ++i) rstd[i] = t;
        }
        char* orow = p.joined + r * p.joined_rs * 2;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = lane + 64 * i;
            if (c < chunks) {
                V8 y, ucopy = uraw[i], xcopy = xraw[i];
                float yf[8], uf32[8];  // y before it is rounded, u in fp32 (used again only when elements are dropped)
                if (p.silu_u || (!GROUP && p.mul_act != HSTU_MUL_U_NONE)) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float uf = (float)uraw[i][j];
                        const float us = uf * sigmoid_f(uf);
                        float mul = uf;
                        if constexpr (GROUP) {
                            if (p.silu_u) mul = us;
                        } else {
                            if (p.mul_act == HSTU_MUL_U_SIGMOID) mul = sigmoid_f(uf);
                            if (p.mul_act == HSTU_MUL_U_SILU) mul = us;
                        }
                        if (p.silu_u) ucopy[j] = (E)us;
                        uf32[j] = uf;
                        yf[j] = mul * ((v[i][j] - mean[i]) * rstd[i] * w[i][GROUP ? 0 : j] + b[i][GROUP ? 0 : j]);
                        y[j] = (E)yf[j];
                    }
                } else {  // no activation anywhere: the exponentials are not worth computing to be thrown away
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        uf32[j] = (float)uraw[i][j];
                        yf[j] = uf32[j] * ((v[i][j] - mean[i]) * rstd[i] * w[i][GROUP ? 0 : j] + b[i][GROUP ? 0 : j]);
                        y[j] = (E)yf[j];
                    }
                }
                if (p.drop.thresh != 0) {
                    // as the reference: the whole of `joined` goes through dropout, in fp32, before it is rounded
                    if (p.off_u >= 0) {
                        float t[8];
#pragma unroll
                        for (int j = 0; j < 8; ++j) t[j] = p.silu_u ? uf32[j] * sigmoid_f(uf32[j]) : uf32[j];
                        ucopy = dropout8<V8, E>(p.drop, r, p.width, (int64_t)p.off_u + c * 8, t);
                    }
                    if (p.off_x >= 0) xcopy = dropout8<V8, E>(p.drop, r, p.width, (int64_t)p.off_x + c * 8, v[i]);
                    y = dropout8<V8, E>(p.drop, r, p.width, (int64_t)p.off_y + c * 8, yf);
                }
                if (p.off_u >= 0) *(V8*)(orow + ((int64_t)p.off_u + c * 8) * 2) = ucopy;
                if (p.off_x >= 0) *(V8*)(orow + ((int64_t)p.off_x + c * 8) * 2) = xcopy;
                *(V8*)(orow + ((int64_t)p.off_y + c * 8) * 2) = y;
            }
        }
    }
}

// False: the ratio is not in [0, 1).
bool dropout_params(float ratio, uint64_t seed, uint64_t offset, hstu::DropoutParams& d) {
    if (!(ratio >= 0.f && ratio < 1.f)) return false;
    d.seed = seed, d.offset = offset;
    d.thresh = (uint32_t)((double)ratio * 4294967296.0);
    d.scale = 1.0f / (1.0f - ratio);
    return true;
}

int output_blocks(const HstuOutputArgs* a) {
    if (a->group_norm) return (a->concat_u && a->concat_x) ? 3 : 1;
    return 1 + (a->concat_u ? 1 : 0) + (a->concat_x ? 1 : 0);
}

int launch_norm_mul(const HstuOutputArgs* a, void* joined, int64_t joined_rs, hipStream_t stream);

// path = 2: which shapes the concatenating GEMM kernel takes, and what the norm-multiply kernel has to leave for it.
bool output_fused_shape(const HstuOutputArgs* a) {
    const int64_t d = (int64_t)a->heads * a->linear_dim;
    if (a->d_out < hstu::kOutWgCols || a->d_out % hstu::kOutWgCols != 0 || a->d_out > 8192) return false;
    if (d < 64 || d > 4096 || (d & 63) != 0 || (a->dtype != 0 && a->dtype != 1)) return false;
    if (a->group_norm && a->silu_u && a->concat_u && a->concat_x) return false;  // (SiLU(u) as a block of its own: layer norm only)
    if (a->attn_row_stride >= (1 << 22) || a->u_row_stride >= (1 << 22)) return false;  // 32-bit byte offsets within a row block
    return true;
}

// The copy of u goes through SiLU: then it is written beside y, as a matrix of its own.
bool output_fused_u_made(const HstuOutputArgs* a) { return !a->group_norm && a->concat_u && a->silu_u; }

// path = 0: the concatenating path where it applies and the rows fill the chip (a workgroup takes 256 rows x 256 columns;
// measured against the library path it wins from 32768 rows on: 70 against 77 us there, 37 against 32 us at 2048).
bool output_takes_fused(const HstuOutputArgs* a) {
    return a->path == 2 || (a->path == 0 && a->rows >= 32768 && a->dropout_ratio == 0.f && output_fused_shape(a));
}

size_t output_fused_workspace(const HstuOutputArgs* a) {
    const size_t d = (size_t)a->heads * a->linear_dim;
    return ((size_t)a->rows * d * 2 * (output_fused_u_made(a) ? 2 : 1) + 255) & ~(size_t)255;
}

template <class TT, bool BIAS>
int launch_output_gemm_t(const hstu::OutputGemmParams& p, hipStream_t stream) {
    auto kern = hstu::hstu_output_gemm_kernel<TT, BIAS>;
    // (a function attribute belongs to the device it was set on: one flag per device)
    static bool attr_done[64];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev >= 64) dev = -1;
    if (dev < 0 || !attr_done[dev]) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, hstu::kOutLds);
        if (e != hipSuccess) {
            snprintf(g_last_error, sizeof(g_last_error), "hipFuncSetAttribute: %s", hipGetErrorString(e));
            return -7;
        }
        if (dev >= 0) attr_done[dev] = true;
    }
    const long long grid = hstu::output_gemm_grid(p.rows, p.n);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(hstu::kOutWaves * 64), hstu::kOutLds, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(g_last_error, sizeof(g_last_error), "output GEMM kernel launch: %s", hipGetErrorString(e));
        return -7;
    }
    return 0;
}

// The caller has checked output_fused_shape(a), the pointers of x, output_weight, out and the size of the workspace.
// y (and SiLU(u) where it is a block) go to the workspace; u and attn are read by the GEMM where they are.
int launch_output_fused(const HstuOutputArgs* a, hipStream_t stream) {
    const int d = a->heads * a->linear_dim;
    const bool u_made = output_fused_u_made(a);
    const int blocks = output_blocks(a);
    const bool cu = blocks == 3 || (!a->group_norm && a->concat_u), cx = blocks == 3 || (!a->group_norm && a->concat_x);
    HstuOutputArgs made = *a;
    made.concat_u = u_made ? 1 : 0, made.concat_x = 0;
    const int64_t ws_rs = (int64_t)d * (u_made ? 2 : 1);
    int rc = launch_norm_mul(&made, a->workspace, ws_rs, stream);
    if (rc != 0) return rc;
    hstu::OutputGemmParams p;
    int n = 0;
    if (cu) p.src[n] = u_made ? (const char*)a->workspace : (const char*)a->u, p.src_rs[n] = u_made ? ws_rs : a->u_row_stride, ++n;
    if (cx) p.src[n] = (const char*)a->attn, p.src_rs[n] = a->attn_row_stride, ++n;
    p.src[n] = (const char*)a->workspace + (u_made ? (int64_t)d * 2 : 0), p.src_rs[n] = ws_rs, ++n;
    for (int i = n; i < 3; ++i) p.src[i] = p.src[0], p.src_rs[i] = p.src_rs[0];
    p.nsrc = n, p.d = d;
    p.x = (const char*)a->x, p.x_rs = a->x_row_stride, p.w = (const char*)a->output_weight, p.out = (char*)a->out, p.rows = a->rows, p.n = a->d_out;
    p.bias = nullptr, p.n_silu = 0;
    return a->dtype == 0 ? launch_output_gemm_t<hstu::Bf16, false>(p, stream) : launch_output_gemm_t<hstu::Fp16, false>(p, stream);
}

int launch_norm_mul(const HstuOutputArgs* a, void* joined, int64_t joined_rs, hipStream_t stream) {
    if (a->rows < 0 || a->heads <= 0 || a->linear_dim <= 0) return -5;
    const int64_t d64 = (int64_t)a->heads * a->linear_dim;
    if (d64 > 4096 || (d64 & 7) != 0) return -5;
    const int d = (int)d64, blocks = output_blocks(a);
    if (a->attn_row_stride < d || a->u_row_stride < d || joined_rs < (int64_t)blocks * d) return -5;
    if (((a->attn_row_stride | a->u_row_stride | joined_rs) & 7) != 0) return -4;
    if (a->dtype != 0 && a->dtype != 1) return -2;
    if (a->mul_u_activation < 0 || a->mul_u_activation > 2) return -5;
    int group_lanes = 0;
    if (a->group_norm) {
        group_lanes = a->linear_dim / 8;
        if ((a->linear_dim & 7) != 0 || group_lanes > 64 || (group_lanes & (group_lanes - 1)) != 0) return -6;
    }
    if (a->rows == 0) return 0;
    if (!a->attn || !a->u || !a->norm_weight || !a->norm_bias || !joined) return -1;
    if ((((uintptr_t)a->attn | (uintptr_t)a->u | (uintptr_t)joined) & 15) != 0) return -4;
    if (!a->group_norm && (((uintptr_t)a->norm_weight | (uintptr_t)a->norm_bias) & 15) != 0) return -4;
    NormMulParams p;
    p.attn = (const char*)a->attn, p.u = (const char*)a->u, p.weight = (const char*)a->norm_weight, p.bias = (const char*)a->norm_bias;
    p.joined = (char*)joined;
    p.attn_rs = a->attn_row_stride, p.u_rs = a->u_row_stride, p.joined_rs = joined_rs, p.rows = a->rows;
    p.eps = a->norm_eps, p.d = d, p.group_lanes = group_lanes;
    const bool cu = blocks == 3 || (!a->group_norm && a->concat_u), cx = blocks == 3 || (!a->group_norm && a->concat_x);
    p.off_u = cu ? 0 : -1;
    p.off_x = cx ? (cu ? d : 0) : -1;
    p.off_y = (blocks - 1) * d;
    p.silu_u = a->silu_u ? 1 : 0, p.mul_act = a->mul_u_activation;
    p.width = (int64_t)blocks * d;
    if (!dropout_params(a->dropout_ratio, a->dropout_seed, a->dropout_offset, p.drop)) return -5;
    long long wgs = (a->rows + 3) / 4;
    if (wgs > 256 * 16) wgs = 256 * 16;
    const int nch = (d / 8 + 63) / 64;
#define HSTU_NM(V8, N, G) hipLaunchKernelGGL((hstu_norm_mul_kernel<V8, N, G>), dim3((unsigned)wgs), dim3(256), 0, stream, p)
#define HSTU_NM_N(V8, G)                                                                                                \
    do {                                                                                                                \
        if (nch <= 1) HSTU_NM(V8, 1, G); else if (nch <= 2) HSTU_NM(V8, 2, G); else if (nch <= 4) HSTU_NM(V8, 4, G); else HSTU_NM(V8, 8, G); \
    } while (0)
    if (a->dtype == 0) {
        if (a->group_norm) HSTU_NM_N(bf16x8_t, true); else HSTU_NM_N(bf16x8_t, false);
    } else {
        if (a->group_norm) HSTU_NM_N(f16x8_t, true); else HSTU_NM_N(f16x8_t, false);
    }
#undef HSTU_NM_N
#undef HSTU_NM
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(g_last_error, sizeof(g_last_error), "norm-mul kernel launch: %s", hipGetErrorString(e));
        return -7;
    }
    return 0;
}

// ---- hipBLASLt: out[rows, n] = epilogue(act[rows, k] @ W[k, n] (+ bias) (+ residual)) ----------------------------------
// Row-major out[rows, n] with row stride ldd is the column-major matrix D[n, rows]; D = A * B with A = W seen
// column-major ([n, k], leading dimension ldw) and B = act seen column-major ([k, rows], leading dimension ldact).
// The bias runs along D's rows, which is what the BIAS epilogues broadcast; the residual is the C operand (beta = 1).
constexpr size_t kGemmScratch = 64u << 20;
enum GemmEpilogue { kEpiNone = 0, kEpiBias = 1, kEpiBiasSilu = 2 };

constexpr int kGemmCandidates = 16;

struct GemmPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr, d = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    // the library's other proposals for this problem, until one call has timed them (see gemm())
    hipblasLtMatmulHeuristicResult_t candidates[kGemmCandidates];
    int ncandidates = 0;
    bool tuned = false;
    long long rows = -1;        // what the layouts b, c, d are built for at the moment
    long long algo_rows = -1;   // what the heuristic was asked about
};

// The number of rows (the total length of a jagged batch) changes from batch to batch, so plans are kept per size class of
// it: the power of two below it and the two bits after that (classes a factor 1.19 .. 1.25 wide, at most 4 per octave).
// That bounds the table by the number of distinct layer shapes times ~130, and one heuristic query serves every batch
// of a class; the three layouts that hold the row count are rebuilt when it differs from the previous call's.
int rows_class(long long rows) {
    const int e = 63 - __builtin_clzll((unsigned long long)rows);
    return e * 4 + (e >= 2 ? (int)((rows >> (e - 2)) & 3) : 0);
}

struct GemmShape {
    long long ldw, ldact, ldres, ldd;
    int rows_class, k, n, dtype, epi, device;
    bool operator<(const GemmShape& o) const {
        return std::tie(rows_class, ldw, ldact, ldres, ldd, k, n, dtype, epi, device) <
               std::tie(o.rows_class, o.ldw, o.ldact, o.ldres, o.ldd, o.k, o.n, o.dtype, o.epi, o.device);
    }
};

std::mutex g_mutex;
hipblasLtHandle_t g_handle = nullptr;
std::map<GemmShape, GemmPlan> g_plans;

int blaslt_fail(const char* what, hipblasStatus_t st) {
    snprintf(g_last_error, sizeof(g_last_error), "%s: hipBLASLt status %d", what, (int)st);
    return HSTU_LINEAR_ERR_BLASLT;
}

// `residual` (row stride ldres) may be null: then ldres must be 0 and beta is 0.
int gemm(const void* act, int64_t ldact, const void* weight, int64_t ldw, const void* bias, const void* residual, int64_t ldres,
         void* out, int64_t ldd, int64_t rows, int k, int n, int dtype, int epi, void* scratch, hipStream_t stream) {
    if (n == 0 || rows == 0) return 0;
    std::lock_guard<std::mutex> lock(g_mutex);
    hipblasStatus_t st;
    if (!g_handle && (st = hipblasLtCreate(&g_handle)) != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtCreate", st);
    int dev = 0;
    (void)hipGetDevice(&dev);
    const GemmShape key{(long long)ldw, (long long)ldact, (long long)ldres, (long long)ldd, rows_class(rows), k, n, dtype, epi, dev};
    const hipDataType t = dtype == 0 ? HIP_R_16BF : HIP_R_16F;
    auto set_rows = [&](GemmPlan& pl) -> hipblasStatus_t {
        if (pl.rows == rows) return HIPBLAS_STATUS_SUCCESS;
        for (hipblasLtMatrixLayout_t* l : {&pl.b, &pl.c, &pl.d})
            if (*l) (void)hipblasLtMatrixLayoutDestroy(*l), *l = nullptr;
        pl.rows = -1;
        hipblasStatus_t s;
        if ((s = hipblasLtMatrixLayoutCreate(&pl.b, t, k, rows, ldact)) != HIPBLAS_STATUS_SUCCESS ||
            (s = hipblasLtMatrixLayoutCreate(&pl.c, t, n, rows, residual ? ldres : ldd)) != HIPBLAS_STATUS_SUCCESS ||
            (s = hipblasLtMatrixLayoutCreate(&pl.d, t, n, rows, ldd)) != HIPBLAS_STATUS_SUCCESS)
            return s;
        pl.rows = rows;
        return HIPBLAS_STATUS_SUCCESS;
    };
    auto ask_heuristic = [&](GemmPlan& pl) -> hipblasStatus_t {
        hipblasLtMatmulPreference_t pref;
        hipblasStatus_t s;
        if ((s = hipblasLtMatmulPreferenceCreate(&pref)) != HIPBLAS_STATUS_SUCCESS) return s;
        const uint64_t max_ws = kGemmScratch;
        hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
        int found = 0;
        s = hipblasLtMatmulAlgoGetHeuristic(g_handle, pl.desc, pl.a, pl.b, pl.c, pl.d, pref, kGemmCandidates, pl.candidates, &found);
        hipblasLtMatmulPreferenceDestroy(pref);
        if (s == HIPBLAS_STATUS_SUCCESS && found < 1) s = HIPBLAS_STATUS_NOT_SUPPORTED;
        if (s != HIPBLAS_STATUS_SUCCESS) return s;
        pl.ncandidates = found;
        pl.algo = pl.candidates[0].algo;
        pl.workspace = pl.candidates[0].workspaceSize;
        pl.algo_rows = rows;
        pl.tuned = false;
        return s;
    };
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        GemmPlan pl;
        if ((st = hipblasLtMatmulDescCreate(&pl.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F)) != HIPBLAS_STATUS_SUCCESS)
            return blaslt_fail("hipblasLtMatmulDescCreate", st);
        if (epi != kEpiNone) {
            const hipblasLtEpilogue_t e = epi == kEpiBiasSilu ? HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT : HIPBLASLT_EPILOGUE_BIAS;
            st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &e, sizeof(e));
            if (st == HIPBLAS_STATUS_SUCCESS) {
                const int32_t bt = (int32_t)t;
                st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt));
            }
            // the bias pointer takes part in the heuristic query; it is set again for every call below
            if (st == HIPBLAS_STATUS_SUCCESS)
                st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
            if (st != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtMatmulDescSetAttribute", st);
        }
        if ((st = hipblasLtMatrixLayoutCreate(&pl.a, t, n, k, ldw)) != HIPBLAS_STATUS_SUCCESS || (st = set_rows(pl)) != HIPBLAS_STATUS_SUCCESS)
            return blaslt_fail("hipblasLtMatrixLayoutCreate", st);
        if ((st = ask_heuristic(pl)) != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtMatmulAlgoGetHeuristic", st);
        it = g_plans.emplace(key, pl).first;
    }
    GemmPlan& pl = it->second;
    if ((st = set_rows(pl)) != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtMatrixLayoutCreate", st);
    if (epi != kEpiNone) {
        st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
        if (st != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("bias pointer", st);
    }
    const float one = 1.0f, beta = residual ? 1.0f : 0.0f;
    // With HSTU_LINEAR_TUNING=1 in the environment the first call that may do so times every proposal of the library on the
    // caller's own operands (as the reference's Triton kernels autotune on first use) and keeps the fastest if it beats the
    // library's first choice by 3 %; every proposal computes the same product, so `out` ends up right whichever ran last.
    // Off by default: measured on the two shapes of the benchmark, the proposals lie within +-4 % of each other and the
    // winner of a back-to-back timing is not reliably the winner between the other kernels of a layer (-6 % for the
    // v|q|k product, +2 % for the output projection).  Never while the stream is being captured into a graph (events
    // cannot be waited for), and not when the product accumulates onto its own output.
    if (!pl.tuned && pl.ncandidates > 1 && getenv("HSTU_LINEAR_TUNING") != nullptr) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        const bool capturing = hipStreamIsCapturing(stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone;
        if (!capturing && residual != out) {
            hipEvent_t e0 = nullptr, e1 = nullptr;
            if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
                float best = 0.f, first = 0.f;
                int best_i = -1;
                // bring the clocks and the caches to where a running loop has them before anything is timed
                for (int rep = 0; rep < 8; ++rep)
                    (void)hipblasLtMatmul(g_handle, pl.desc, &one, weight, pl.a, act, pl.b, &beta, residual ? residual : out, pl.c, out,
                                          pl.d, &pl.candidates[0].algo, scratch, pl.candidates[0].workspaceSize, stream);
                for (int i = 0; i < pl.ncandidates; ++i) {
                    if (pl.candidates[i].workspaceSize > kGemmScratch) continue;
                    float fastest = 0.f;
                    bool ok = true;
                    for (int rep = 0; rep < 5 && ok; ++rep) {
                        (void)hipEventRecord(e0, stream);
                        st = hipblasLtMatmul(g_handle, pl.desc, &one, weight, pl.a, act, pl.b, &beta, residual ? residual : out, pl.c, out,
                                             pl.d, &pl.candidates[i].algo, scratch, pl.candidates[i].workspaceSize, stream);
                        (void)hipEventRecord(e1, stream);
                        float ms = 0.f;
                        ok = st == HIPBLAS_STATUS_SUCCESS && hipEventSynchronize(e1) == hipSuccess &&
                             hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
                        if (ok && rep > 0 && (fastest == 0.f || ms < fastest)) fastest = ms;  // the first run warms up
                    }
                    if (ok && i == 0) first = fastest;
                    if (ok && fastest > 0.f && (best_i < 0 || fastest < best)) best = fastest, best_i = i;
                }
                // the library's own first choice stays unless another one is clearly (3 %) faster
                if (best_i > 0 && first > 0.f && best > 0.97f * first) best_i = 0;
                if (best_i >= 0) {
                    pl.algo = pl.candidates[best_i].algo;
                    pl.workspace = pl.candidates[best_i].workspaceSize;
                }
                pl.tuned = true;
            }
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
        }
    }
    st = hipblasLtMatmul(g_handle, pl.desc, &one, weight, pl.a, act, pl.b, &beta, residual ? residual : out, pl.c, out, pl.d, &pl.algo,
                         scratch, kGemmScratch, stream);  // all of it: the need may grow with the rows within a size class
    if (st != HIPBLAS_STATUS_SUCCESS && pl.algo_rows != rows) {
        // the choice made for another row count of the same size class does not take this one: ask for this one
        if ((st = ask_heuristic(pl)) != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtMatmulAlgoGetHeuristic", st);
        st = hipblasLtMatmul(g_handle, pl.desc, &one, weight, pl.a, act, pl.b, &beta, residual ? residual : out, pl.c, out, pl.d,
                             &pl.algo, scratch, kGemmScratch, stream);
    }
    if (st != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtMatmul", st);
    return 0;
}

bool uqvk_fused_shape(const HstuUqvkArgs* a) {
    const int n_u = a->hidden_dim * a->heads;
    const int n_out = (2 * a->hidden_dim + 2 * a->attn_dim) * a->heads;
    return (a->d_model == 128 || a->d_model == 256 || a->d_model == 384 || a->d_model == 512) && n_u % 128 == 0 && n_out % 128 == 0 &&
           (a->dtype == 0 || a->dtype == 1);
}

template <class TT, int KT>
int launch_uqvk_fused(const hstu::UqvkFusedParams& p, hipStream_t stream) {
    auto kern = hstu::hstu_uqvk_fused_kernel<TT, KT>;
    // (a function attribute belongs to the device it was set on: one flag per device)
    static bool attr_done[64];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev >= 64) dev = -1;
    if (dev < 0 || !attr_done[dev]) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, hstu::kUqvkLds);
        if (e != hipSuccess) {
            snprintf(g_last_error, sizeof(g_last_error), "hipFuncSetAttribute: %s", hipGetErrorString(e));
            return -7;
        }
        if (dev >= 0) attr_done[dev] = true;
    }
    constexpr int kRows = hstu::kUqvkWaves * hstu::kUqvkRowsPerWave;
    const long long grid = (p.rows + kRows - 1) / kRows;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(hstu::kUqvkWaves * 64), hstu::kUqvkLds, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(g_last_error, sizeof(g_last_error), "fused uqvk kernel launch: %s", hipGetErrorString(e));
        return -7;
    }
    return 0;
}

template <class TT>
int launch_uqvk_fused_k(const hstu::UqvkFusedParams& p, int d_model, hipStream_t stream) {
    switch (d_model) {
        case 128: return launch_uqvk_fused<TT, 2>(p, stream);
        case 256: return launch_uqvk_fused<TT, 4>(p, stream);
        case 384: return launch_uqvk_fused<TT, 6>(p, stream);
        default: return launch_uqvk_fused<TT, 8>(p, stream);
    }
}

size_t normed_bytes(const HstuUqvkArgs* a) { return (((size_t)a->rows * a->d_model * 2) + 255) & ~(size_t)255; }
size_t joined_bytes(const HstuOutputArgs* a) {
    return (((size_t)a->rows * output_blocks(a) * a->heads * a->linear_dim * 2) + 255) & ~(size_t)255;
}

}  // namespace

extern "C" {

const char* hstu_linear_last_error(void) { return g_last_error; }

int hstu_linear_version(void) { return 101; }

size_t hstu_uqvk_workspace_bytes(const HstuUqvkArgs* a) {
    if (!a || a->rows <= 0 || a->d_model <= 0) return 0;
    if (a->path != 1 && a->path != 3 && a->heads > 0 && a->attn_dim > 0 && a->hidden_dim > 0 && uqvk_fused_shape(a)) return 0;
    return normed_bytes(a) + kGemmScratch;
}

int hstu_uqvk_layer_norm(const void* x, int64_t x_row_stride, const void* weight, const void* bias, float eps, void* out,
                         int64_t out_row_stride, int64_t rows, int32_t d_model, int32_t dtype, void* stream) {
    g_last_error[0] = 0;
    return launch_layer_norm(x, x_row_stride, weight, bias, eps, out, out_row_stride, rows, d_model, dtype, (hipStream_t)stream);
}

int hstu_uqvk_forward(const HstuUqvkArgs* a, void* stream_) {
    g_last_error[0] = 0;
    if (!a) return -1;
    if (a->rows < 0 || a->heads <= 0 || a->attn_dim <= 0 || a->hidden_dim <= 0 || a->d_model <= 0) return -5;
    if (a->rows == 0) return 0;
    if (a->path < 0 || a->path > 3) return -5;
    if (!a->uvqk_weight || !a->uvqk_bias || !a->uvqk) return -1;
    if (a->rows > 0x7fffffffLL) return -5;
    hipStream_t stream = (hipStream_t)stream_;
    const int n_u = a->hidden_dim * a->heads;
    const int n_out = (2 * a->hidden_dim + 2 * a->attn_dim) * a->heads;
    if ((n_u & 7) != 0 || (n_out & 7) != 0) return -4;  // column blocks start on 16-byte boundaries
    const bool fused = a->path != 1 && a->path != 3 && uqvk_fused_shape(a);
    if (a->path == 2 && !fused) return -6;
    if (a->qkv_fp8 && !fused) {
        snprintf(g_last_error, sizeof(g_last_error), "the e4m3 copy of v | q | k is written by the fused kernel only (path 0 or 2, d_model 128 .. 512)");
        return -6;
    }
    // the layer-norm kernel + the hand-written GEMM of the output projection in its bias / SiLU form, on request only
    // (path 3): with 8 column blocks per row block and a depth of 16 .. 32 tiles it is slower than the library path
    // (2.23 against 1.72 ms at d_model 512, 3.15 against 2.42 ms at 1024; 524288 rows, 2048 columns)
    const bool gemm_shape = (a->d_model & 63) == 0 && a->d_model >= 64 && a->d_model <= 4096 && n_out % hstu::kOutWgCols == 0 &&
                            n_u % hstu::kOutWgCols == 0 && n_out <= 8192 && (a->dtype == 0 || a->dtype == 1);
    if (a->path == 3 && !gemm_shape) {
        snprintf(g_last_error, sizeof(g_last_error), "path 3 takes d_model a multiple of 64 and hidden_dim * heads, n_out multiples of 256");
        return -6;
    }
    const bool hand_gemm = a->path == 3;
    if (fused) {
        if (!a->x || !a->norm_weight || !a->norm_bias) return -1;
        if (a->x_row_stride < a->d_model || (a->x_row_stride & 7) != 0) return -5;
        const uintptr_t ptrs = (uintptr_t)a->x | (uintptr_t)a->norm_weight | (uintptr_t)a->norm_bias | (uintptr_t)a->uvqk_weight |
                               (uintptr_t)a->uvqk_bias | (uintptr_t)a->uvqk;
        if ((ptrs & 15) != 0) return -4;
        hstu::UqvkFusedParams p;
        p.x = (const char*)a->x, p.x_rs = a->x_row_stride;
        p.norm_weight = (const char*)a->norm_weight, p.norm_bias = (const char*)a->norm_bias, p.eps = a->norm_eps;
        p.w = (const char*)a->uvqk_weight, p.bias = (const char*)a->uvqk_bias, p.out = (char*)a->uvqk;
        p.rows = a->rows, p.n_out = n_out, p.n_silu = n_u;
        p.out8 = (unsigned char*)a->qkv_fp8, p.absmax = (unsigned*)a->qkv_absmax, p.n_attn = a->attn_dim * a->heads;
        if (a->qkv_fp8) {
            if (!a->qkv_absmax) return -1;
            if (((uintptr_t)a->qkv_fp8 & 15) != 0 || ((uintptr_t)a->qkv_absmax & 3) != 0) return -4;
            const float sc[3] = {a->v_scale, a->q_scale, a->k_scale};
            for (int i = 0; i < 3; ++i) {
                if (!(sc[i] > 0.f)) return -5;
                p.inv_scale[i] = 1.0f / sc[i];
            }
        }
        return a->dtype == 0 ? launch_uqvk_fused_k<hstu::Bf16>(p, a->d_model, stream) : launch_uqvk_fused_k<hstu::Fp16>(p, a->d_model, stream);
    }
    if (!a->workspace) return -1;
    if ((size_t)a->workspace_bytes < hstu_uqvk_workspace_bytes(a) || ((uintptr_t)a->workspace & 255) != 0) return -4;
    void* normed = a->workspace;
    void* scratch = (char*)a->workspace + normed_bytes(a);
    int rc = launch_layer_norm(a->x, a->x_row_stride, a->norm_weight, a->norm_bias, a->norm_eps, normed, a->d_model, a->rows,
                               a->d_model, a->dtype, stream);
    if (rc != 0) return rc;
    if (hand_gemm) {
        if ((((uintptr_t)a->uvqk_weight | (uintptr_t)a->uvqk_bias | (uintptr_t)a->uvqk) & 15) != 0) return -4;
        hstu::OutputGemmParams p;
        for (int i = 0; i < 3; ++i) p.src[i] = (const char*)normed, p.src_rs[i] = a->d_model;
        p.nsrc = 1, p.d = a->d_model, p.x = nullptr, p.x_rs = 0;
        p.w = (const char*)a->uvqk_weight, p.out = (char*)a->uvqk, p.rows = a->rows, p.n = n_out;
        p.bias = (const char*)a->uvqk_bias, p.n_silu = n_u;
        return a->dtype == 0 ? launch_output_gemm_t<hstu::Bf16, true>(p, stream) : launch_output_gemm_t<hstu::Fp16, true>(p, stream);
    }
    // u columns with SiLU in the epilogue, then v | q | k with the bias only
    const char* w = (const char*)a->uvqk_weight;
    const char* b = (const char*)a->uvqk_bias;
    char* o = (char*)a->uvqk;
    rc = gemm(normed, a->d_model, w, n_out, b, nullptr, 0, o, n_out, a->rows, a->d_model, n_u, a->dtype, kEpiBiasSilu, scratch, stream);
    if (rc != 0) return rc;
    return gemm(normed, a->d_model, w + (int64_t)n_u * 2, n_out, b + (int64_t)n_u * 2, nullptr, 0, o + (int64_t)n_u * 2, n_out, a->rows,
                a->d_model, n_out - n_u, a->dtype, kEpiBias, scratch, stream);
}

size_t hstu_output_workspace_bytes(const HstuOutputArgs* a) {
    if (!a || a->rows <= 0 || a->heads <= 0 || a->linear_dim <= 0) return 0;
    if (output_takes_fused(a)) return output_fused_shape(a) ? output_fused_workspace(a) : 0;
    return joined_bytes(a) + kGemmScratch;
}

int hstu_output_norm_mul(const HstuOutputArgs* a, void* joined, int64_t joined_row_stride, void* stream) {
    g_last_error[0] = 0;
    if (!a) return -1;
    return launch_norm_mul(a, joined, joined_row_stride, (hipStream_t)stream);
}

int hstu_output_dropout_mask(float ratio, uint64_t seed, uint64_t offset, int64_t rows, int64_t width, void* keep, void* stream) {
    g_last_error[0] = 0;
    hstu::DropoutParams d;
    if (rows < 0 || width < 0 || (width & 7) != 0 || !dropout_params(ratio, seed, offset, d)) return -5;
    if (rows == 0 || width == 0) return 0;
    if (!keep) return -1;
    if (((uintptr_t)keep & 3) != 0) return -4;
    const int64_t groups = rows * width / 4;
    long long wgs = (groups + 255) / 256;
    if (wgs > 256 * 16) wgs = 256 * 16;
    hipLaunchKernelGGL(hstu_dropout_mask_kernel, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream, d, groups, (unsigned char*)keep);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(g_last_error, sizeof(g_last_error), "dropout mask kernel launch: %s", hipGetErrorString(e));
        return -7;
    }
    return 0;
}

int hstu_output_forward(const HstuOutputArgs* a, void* stream_) {
    g_last_error[0] = 0;
    if (!a) return -1;
    if (a->rows < 0 || a->heads <= 0 || a->linear_dim <= 0 || a->d_out <= 0 || (a->d_out & 7) != 0) return -5;
    if (a->rows > 0x7fffffffLL || a->x_row_stride < a->d_out || (a->x_row_stride & 7) != 0) return -5;
    if (a->rows == 0) return 0;
    if (a->path < 0 || a->path > 2) return -5;
    if (!a->x || !a->output_weight || !a->out) return -1;
    if ((((uintptr_t)a->x | (uintptr_t)a->output_weight | (uintptr_t)a->out) & 15) != 0) return -4;
    hipStream_t stream = (hipStream_t)stream_;
    if (a->path == 2 && !output_fused_shape(a)) {
        snprintf(g_last_error, sizeof(g_last_error), "the concatenating output kernel takes d_out a multiple of 256 and heads * linear_dim a multiple "
                 "of 64 up to 4096, row strides below 2^22 (and, with group norm, no SiLU on a copied u)");
        return -6;
    }
    if (a->dropout_ratio != 0.f && a->path == 2) {
        snprintf(g_last_error, sizeof(g_last_error), "the concatenating output kernel reads u and attn where they are and cannot drop their "
                 "elements: dropout runs on the library path (path 0 or 1)");
        return -6;
    }
    if (output_takes_fused(a)) {
        if (!a->workspace) return -1;
        if ((size_t)a->workspace_bytes < output_fused_workspace(a) || ((uintptr_t)a->workspace & 255) != 0) return -4;
        return launch_output_fused(a, stream);
    }
    if (!a->workspace) return -1;
    if ((size_t)a->workspace_bytes < joined_bytes(a) + kGemmScratch || ((uintptr_t)a->workspace & 255) != 0) return -4;
    const int k = output_blocks(a) * a->heads * a->linear_dim;
    void* joined = a->workspace;
    void* scratch = (char*)a->workspace + joined_bytes(a);
    int rc = launch_norm_mul(a, joined, k, stream);
    if (rc != 0) return rc;
    return gemm(joined, k, a->output_weight, a->d_out, nullptr, a->x, a->x_row_stride, a->out, a->d_out, a->rows, k, a->d_out, a->dtype,
                kEpiNone, scratch, stream);
}

}  // extern "C"
