// C ABI of libhstu_uqvk.so: layer norm kernel + hipBLASLt GEMMs with fused bias / SiLU epilogues.
// Declarations and the reference interface they replace are in include/hstu_uqvk.h.
#include "hstu_uqvk.h"

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdio>
#include <map>
#include <mutex>
#include <tuple>

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

// ---- hipBLASLt: out[:, c0:c0+n] = act(normed @ W[:, c0:c0+n] + bias[c0:c0+n]) ------------------------------------
// Row-major out[rows, n_out] is the column-major matrix D[n_out, rows]; D = A * B with A = W seen column-major
// ([n, d_model], leading dimension n_out) and B = normed seen column-major ([d_model, rows]).  The bias runs along
// D's rows, which is what the BIAS epilogues broadcast.
constexpr size_t kGemmScratch = 64u << 20;

struct GemmPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, d = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
};

std::mutex g_mutex;
hipblasLtHandle_t g_handle = nullptr;
std::map<std::tuple<int, long long, int, int, int, int>, GemmPlan> g_plans;  // (device, rows, d_model, n, n_out, dtype*2+silu)

int blaslt_fail(const char* what, hipblasStatus_t st) {
    snprintf(g_last_error, sizeof(g_last_error), "%s: hipBLASLt status %d", what, (int)st);
    return HSTU_UQVK_ERR_BLASLT;
}

int gemm_part(const void* normed, const char* weight, const char* bias, char* out, int64_t rows, int d_model, int n, int n_out,
              int c0, int dtype, bool silu, void* scratch, hipStream_t stream) {
    if (n == 0 || rows == 0) return 0;
    std::lock_guard<std::mutex> lock(g_mutex);
    hipblasStatus_t st;
    if (!g_handle && (st = hipblasLtCreate(&g_handle)) != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtCreate", st);
    int dev = 0;
    (void)hipGetDevice(&dev);
    const auto key = std::make_tuple(dev, (long long)rows, d_model, n, n_out, dtype * 2 + (silu ? 1 : 0));
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        GemmPlan pl;
        const hipDataType t = dtype == 0 ? HIP_R_16BF : HIP_R_16F;
        if ((st = hipblasLtMatmulDescCreate(&pl.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F)) != HIPBLAS_STATUS_SUCCESS)
            return blaslt_fail("hipblasLtMatmulDescCreate", st);
        const hipblasLtEpilogue_t epi = silu ? HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT : HIPBLASLT_EPILOGUE_BIAS;
        st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi));
        if (st == HIPBLAS_STATUS_SUCCESS) {
            const int32_t bt = (int32_t)t;
            st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt));
        }
        if (st != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtMatmulDescSetAttribute", st);
        if ((st = hipblasLtMatrixLayoutCreate(&pl.a, t, n, d_model, n_out)) != HIPBLAS_STATUS_SUCCESS ||
            (st = hipblasLtMatrixLayoutCreate(&pl.b, t, d_model, rows, d_model)) != HIPBLAS_STATUS_SUCCESS ||
            (st = hipblasLtMatrixLayoutCreate(&pl.d, t, n, rows, n_out)) != HIPBLAS_STATUS_SUCCESS)
            return blaslt_fail("hipblasLtMatrixLayoutCreate", st);
        // the bias pointer takes part in the heuristic query; it is set again for every call below
        const void* bp = bias + (int64_t)c0 * 2;
        st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp));
        if (st != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("bias pointer", st);
        hipblasLtMatmulPreference_t pref;
        if ((st = hipblasLtMatmulPreferenceCreate(&pref)) != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("preference", st);
        const uint64_t max_ws = kGemmScratch;
        hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
        hipblasLtMatmulHeuristicResult_t res[1];
        int found = 0;
        st = hipblasLtMatmulAlgoGetHeuristic(g_handle, pl.desc, pl.a, pl.b, pl.d, pl.d, pref, 1, res, &found);
        hipblasLtMatmulPreferenceDestroy(pref);
        if (st != HIPBLAS_STATUS_SUCCESS || found < 1) return blaslt_fail("hipblasLtMatmulAlgoGetHeuristic", st);
        pl.algo = res[0].algo;
        pl.workspace = res[0].workspaceSize;
        it = g_plans.emplace(key, pl).first;
    }
    GemmPlan& pl = it->second;
    const void* bp = bias + (int64_t)c0 * 2;
    st = hipblasLtMatmulDescSetAttribute(pl.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp));
    if (st != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("bias pointer", st);
    const float one = 1.0f, zero = 0.0f;
    char* dptr = out + (int64_t)c0 * 2;
    st = hipblasLtMatmul(g_handle, pl.desc, &one, weight + (int64_t)c0 * 2, pl.a, normed, pl.b, &zero, dptr, pl.d, dptr, pl.d, &pl.algo,
                         scratch, pl.workspace, stream);
    if (st != HIPBLAS_STATUS_SUCCESS) return blaslt_fail("hipblasLtMatmul", st);
    return 0;
}

size_t normed_bytes(const HstuUqvkArgs* a) { return (((size_t)a->rows * a->d_model * 2) + 255) & ~(size_t)255; }

}  // namespace

extern "C" {

const char* hstu_uqvk_last_error(void) { return g_last_error; }

size_t hstu_uqvk_workspace_bytes(const HstuUqvkArgs* a) {
    if (!a || a->rows <= 0 || a->d_model <= 0) return 0;
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
    if (!a->uvqk_weight || !a->uvqk_bias || !a->uvqk || !a->workspace) return -1;
    if ((size_t)a->workspace_bytes < hstu_uqvk_workspace_bytes(a) || ((uintptr_t)a->workspace & 255) != 0) return -4;
    if (a->rows > 0x7fffffffLL) return -5;
    hipStream_t stream = (hipStream_t)stream_;
    const int n_u = a->hidden_dim * a->heads;
    const int n_out = (2 * a->hidden_dim + 2 * a->attn_dim) * a->heads;
    if ((n_u & 7) != 0 || (n_out & 7) != 0) return -4;  // column blocks start on 16-byte boundaries
    void* normed = a->workspace;
    void* scratch = (char*)a->workspace + normed_bytes(a);
    int rc = launch_layer_norm(a->x, a->x_row_stride, a->norm_weight, a->norm_bias, a->norm_eps, normed, a->d_model, a->rows,
                               a->d_model, a->dtype, stream);
    if (rc != 0) return rc;
    // u columns with SiLU in the epilogue, then v | q | k with the bias only
    rc = gemm_part(normed, (const char*)a->uvqk_weight, (const char*)a->uvqk_bias, (char*)a->uvqk, a->rows, a->d_model, n_u, n_out, 0,
                   a->dtype, true, scratch, stream);
    if (rc != 0) return rc;
    return gemm_part(normed, (const char*)a->uvqk_weight, (const char*)a->uvqk_bias, (char*)a->uvqk, a->rows, a->d_model, n_out - n_u,
                     n_out, n_u, a->dtype, false, scratch, stream);
}

}  // extern "C"
