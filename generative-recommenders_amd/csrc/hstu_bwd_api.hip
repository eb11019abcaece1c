// C ABI of the backward pass (hstu_hip_mha_bwd): validation and launch of the two kernels of hstu_bwd_kernel.h.
// A translation unit of its own so that it compiles in parallel with the forward kernels.
#include "hstu_hip.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

#include "hstu_bwd_kernel.h"
#include "hstu_bwd_pp_kernel.h"

// defined with the forward entry points (hstu_api.hip); internal to the library
extern "C" __attribute__((visibility("hidden"))) int hstu_hip_device_is_gfx950(void);
extern "C" __attribute__((visibility("hidden"))) void hstu_hip_set_last_error(const char* what, int hip_error);
extern "C" __attribute__((visibility("hidden"))) int hstu_hip_launch_rank(const void* offsets, int offsets_i64, int batch, int* order,
                                                                          void* stream);

namespace {

constexpr int kBwdWaves = 4, kBwdTile = 64, kBwdRows = kBwdWaves * 32;
constexpr int kStoredWaves = 8, kStoredRows = kStoredWaves * 32;  // the dQ kernel that reads stored dS

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Bytes of the dS blocks: (total rows + 32 per sequence) x H x pitch32 x 64, pitch32 = 4 * ceil(max_seq_len / 128).
size_t ds_bytes(const HstuFwdArgs* a) {
    const size_t pitch32 = 4 * (((size_t)a->max_seq_len + 127) / 128);
    return ((size_t)a->total_q + 32 * (size_t)a->batch) * (size_t)a->heads * pitch32 * 64;
}

template <class TT, int DQK, int DV, bool STORE>
auto key_stationary_kernel(std::true_type) {
    return hstu::hstu_bwd_dkdv_pp_kernel<TT, DQK, DV, STORE>;
}
template <class TT, int DQK, int DV, bool STORE>
auto key_stationary_kernel(std::false_type) {
    return hstu::hstu_bwd_dkdv_kernel<TT, DQK, DV, kBwdWaves, kBwdTile, STORE>;
}

template <class TT, int DQK, int DV>
int launch_bwd(const hstu::BwdParams& bp, hipStream_t stream) {
    // three tile slots for the key-stationary kernel, two for the other; + 64: transposing reads of a 16-wide tile's unused half
    constexpr int smem1 = 3 * kBwdTile * (DQK + DV) * 2 + 64;
    constexpr int smem = 2 * kBwdTile * (DQK + DV) * 2 + 64;
    constexpr int smem3 = 3 * kBwdTile * DQK * 2 + kStoredWaves * 3 * 4096;
    // The key-stationary kernel: with two waves per SIMD where a tile copy gives every copying wave something to do and
    // the byte offsets inside a tile of 64 rows fit its 32-bit arithmetic; the one-wave kernel otherwise.
    constexpr bool kPairedDims = DQK >= 32 && DV >= 32;
    auto k1p = key_stationary_kernel<TT, DQK, DV, false>(std::integral_constant<bool, kPairedDims>{});
    auto k1ps = key_stationary_kernel<TT, DQK, DV, true>(std::integral_constant<bool, kPairedDims>{});
    constexpr int smem1p = kPairedDims ? hstu::bwd_pp_lds_bytes<(DQK < 32 ? 32 : DQK), (DV < 32 ? 32 : DV)>() : 0;
    const bool paired = kPairedDims && bp.f.q_rs < (1 << 22) && bp.do_rs < (1 << 22);
    auto k1 = hstu::hstu_bwd_dkdv_kernel<TT, DQK, DV, kBwdWaves, kBwdTile, false>;
    auto k1s = hstu::hstu_bwd_dkdv_kernel<TT, DQK, DV, kBwdWaves, kBwdTile, true>;
    auto k2 = hstu::hstu_bwd_dq_kernel<TT, DQK, DV, kBwdWaves, kBwdTile>;
    auto k3 = hstu::hstu_bwd_dq_stored_kernel<TT, DQK, kStoredWaves, kBwdTile>;
    // (a function attribute belongs to the device it was set on: one flag per device)
    static bool attr_done[64];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev >= 64) dev = -1;
    if (dev < 0 || !attr_done[dev]) {
        hipError_t e = hipFuncSetAttribute((const void*)k1, hipFuncAttributeMaxDynamicSharedMemorySize, smem1);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)k1s, hipFuncAttributeMaxDynamicSharedMemorySize, smem1);
        if (kPairedDims) {
            if (e == hipSuccess) e = hipFuncSetAttribute((const void*)k1p, hipFuncAttributeMaxDynamicSharedMemorySize, smem1p);
            if (e == hipSuccess) e = hipFuncSetAttribute((const void*)k1ps, hipFuncAttributeMaxDynamicSharedMemorySize, smem1p);
        }
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)k2, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void*)k3, hipFuncAttributeMaxDynamicSharedMemorySize, smem3);
        if (e != hipSuccess) {
            hstu_hip_set_last_error("hipFuncSetAttribute", (int)e);
            return HSTU_ERR_LAUNCH;
        }
        if (dev >= 0) attr_done[dev] = true;
    }
    const unsigned grid = (unsigned)bp.f.slots_per_xcd * 8;
    if (bp.ds) {
        if (paired) hipLaunchKernelGGL(k1ps, dim3(grid), dim3(hstu::kBwdPpWaves * 64), smem1p, stream, bp);
        else hipLaunchKernelGGL(k1s, dim3(grid), dim3(kBwdWaves * 64), smem1, stream, bp);
        hstu::BwdParams b3 = bp;  // the same items in blocks of 256 query rows
        b3.f.num_mb = (bp.f.max_seq_len + kStoredRows - 1) / kStoredRows;
        b3.f.slots_per_xcd = bp.f.pairs_per_xcd * b3.f.num_mb;
        hipLaunchKernelGGL(k3, dim3((unsigned)b3.f.slots_per_xcd * 8), dim3(kStoredWaves * 64), smem3, stream, b3);
    } else {
        if (paired) hipLaunchKernelGGL(k1p, dim3(grid), dim3(hstu::kBwdPpWaves * 64), smem1p, stream, bp);
        else hipLaunchKernelGGL(k1, dim3(grid), dim3(kBwdWaves * 64), smem1, stream, bp);
        hipLaunchKernelGGL(k2, dim3(grid), dim3(kBwdWaves * 64), smem, stream, bp);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        hstu_hip_set_last_error("backward kernel launch", (int)e);
        return HSTU_ERR_LAUNCH;
    }
    return HSTU_OK;
}

template <class TT, int DQK>
int launch_bwd_dv(const hstu::BwdParams& bp, int dv, hipStream_t stream) {
    switch (dv) {
        case 16: return launch_bwd<TT, DQK, 16>(bp, stream);
        case 32: return launch_bwd<TT, DQK, 32>(bp, stream);
        case 64: return launch_bwd<TT, DQK, 64>(bp, stream);
        case 128: return launch_bwd<TT, DQK, 128>(bp, stream);
        default: return HSTU_ERR_BAD_HEAD_DIM;
    }
}

template <class TT>
int launch_bwd_dim(const hstu::BwdParams& bp, int dqk, int dv, hipStream_t stream) {
    switch (dqk) {
        case 16: return launch_bwd_dv<TT, 16>(bp, dv, stream);
        case 32: return launch_bwd_dv<TT, 32>(bp, dv, stream);
        case 64: return launch_bwd_dv<TT, 64>(bp, dv, stream);
        case 128: return launch_bwd_dv<TT, 128>(bp, dv, stream);
        default: return HSTU_ERR_BAD_HEAD_DIM;
    }
}

}  // namespace

extern "C" size_t hstu_hip_mha_bwd_workspace_bytes(const HstuFwdArgs* a) {
    if (!a || a->batch <= 0 || a->heads <= 0 || a->max_seq_len <= 0 || a->total_q <= 0) return 0;
    return align256((size_t)a->batch * sizeof(int)) + ds_bytes(a);
}

extern "C" int hstu_hip_mha_bwd(const HstuFwdArgs* a, const HstuBwdGrads* g, void* stream_) {
    if (!a || !g) return HSTU_ERR_NULL_POINTER;
    HstuFwdArgs c = *a;  // the forward's own checks, with the unused output standing in as any aligned pointer
    c.out = const_cast<void*>(a->q);
    c.o_row_stride = c.o_head_stride = 0;
    c.tile_config = 0;
    c.kv_splits = 0;
    int rc = hstu_hip_check_args(&c);
    if (rc != HSTU_OK) return rc;
    if (a->delta_size != 0) return HSTU_ERR_UNSUPPORTED;
    if (a->dtype != HSTU_BF16 && a->dtype != HSTU_FP16) return HSTU_ERR_UNSUPPORTED;
    // the kernels scale by 1 / max_seq_len: a caller with an attn_scale multiplies dout by attn_scale * max_seq_len
    // itself (a per-row factor commutes with everything behind it) and calls with attn_scale = NULL
    if (a->attn_scale) return HSTU_ERR_UNSUPPORTED;
    if (a->total_q == 0 || a->batch == 0) return HSTU_OK;
    if (!g->dout || !g->dq || !g->dk || !g->dv) return HSTU_ERR_NULL_POINTER;
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(g->dout) | reinterpret_cast<uintptr_t>(g->dq) |
                           reinterpret_cast<uintptr_t>(g->dk) | reinterpret_cast<uintptr_t>(g->dv);
    if ((ptrs & 15) != 0) return HSTU_ERR_MISALIGNED;
    const int64_t strides[8] = {g->do_row_stride, g->do_head_stride, g->dq_row_stride, g->dq_head_stride,
                                g->dk_row_stride, g->dk_head_stride, g->dv_row_stride, g->dv_head_stride};
    for (int i = 0; i < 8; ++i)
        if (strides[i] < 0 || (strides[i] & 7) != 0) return HSTU_ERR_MISALIGNED;
    if (!hstu_hip_device_is_gfx950()) return HSTU_ERR_BAD_DEVICE;
    hipStream_t stream = (hipStream_t)stream_;

    hstu::BwdParams bp;
    memset(&bp, 0, sizeof(bp));
    hstu::FwdParams& p = bp.f;
    p.q = (const char*)a->q;
    p.k = (const char*)a->k;
    p.v = (const char*)a->v;
    p.q_rs = a->q_row_stride, p.q_hs = a->q_head_stride;
    p.k_rs = a->k_row_stride, p.k_hs = a->k_head_stride;
    p.v_rs = a->v_row_stride, p.v_hs = a->v_head_stride;
    p.offsets = a->seq_offsets;
    p.targets = a->num_targets;
    p.offsets_i64 = a->seq_offsets_i64;
    p.targets_i64 = a->num_targets_i64;
    p.B = a->batch;
    p.H = a->heads;
    p.max_seq_len = a->max_seq_len;
    p.w = a->max_attn_len;
    p.c = a->contextual_seq_len;
    p.f = a->min_full_attn_seq_len;
    p.kv_splits = 1;
    p.c1 = -a->alpha * 1.4426950408889634f;
    bp.gscale = a->alpha / (float)a->max_seq_len;
    bp.pscale = a->alpha == 0.0f ? 0.0f : -1.0f / ((float)a->max_seq_len * 1.4426950408889634f);
    bp.dout = (const char*)g->dout;
    bp.dq = (char*)g->dq, bp.dk = (char*)g->dk, bp.dv = (char*)g->dv;
    bp.do_rs = g->do_row_stride, bp.do_hs = g->do_head_stride;
    bp.dq_rs = g->dq_row_stride, bp.dq_hs = g->dq_head_stride;
    bp.dk_rs = g->dk_row_stride, bp.dk_hs = g->dk_head_stride;
    bp.dv_rs = g->dv_row_stride, bp.dv_hs = g->dv_head_stride;

    p.num_mb = (a->max_seq_len + kBwdRows - 1) / kBwdRows;
    const long long pairs_per_xcd = ((long long)a->batch * a->heads + 7) / 8;
    const long long slots = pairs_per_xcd * p.num_mb;
    if (slots * 8 > 0x7fffffffLL) return HSTU_ERR_BAD_SHAPE;
    p.pairs_per_xcd = (int)pairs_per_xcd;
    p.slots_per_xcd = (int)slots;

    // `sort_by_length`: long sequences first (their blocks are the long-running ones); needs 4 * batch bytes of workspace
    if (a->sort_by_length && a->batch >= 2 && a->batch <= 8192 && a->workspace &&
        (size_t)a->workspace_bytes >= (size_t)a->batch * sizeof(int)) {
        rc = hstu_hip_launch_rank(a->seq_offsets, a->seq_offsets_i64, a->batch, (int*)a->workspace, stream_);
        if (rc != HSTU_OK) return rc;
        p.order = (const int*)a->workspace;
    }
    // enough workspace for the dS blocks: the key-stationary kernel stores them and dQ is formed from them
    if (a->workspace && (size_t)a->workspace_bytes >= hstu_hip_mha_bwd_workspace_bytes(a) &&
        (reinterpret_cast<uintptr_t>(a->workspace) & 255) == 0) {
        bp.ds = (char*)a->workspace + align256((size_t)a->batch * sizeof(int));
        bp.ds_pitch32 = 4 * ((a->max_seq_len + 127) / 128);
    }
    if (a->dtype == HSTU_BF16) return launch_bwd_dim<hstu::Bf16>(bp, a->dqk, a->dv, stream);
    return launch_bwd_dim<hstu::Fp16>(bp, a->dqk, a->dv, stream);
}
