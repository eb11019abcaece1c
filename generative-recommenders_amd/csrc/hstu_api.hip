// C ABI of libhstu_hip.so: argument validation, kernel selection and launch.
// Declarations and the reference interfaces they replace are in include/hstu_hip.h.
#include "hstu_hip.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <initializer_list>
#include <mutex>

#include "hstu_fwd_kernel.h"
#include "hstu_fwd_pp_kernel.h"
#include "hstu_fwd_stream_kernel.h"
#include "hstu_jagged_kernels.h"

// Scratch area of hstu_hip_mha_fwd_noalloc: what the caller's `workspace` is to hstu_hip_mha_fwd (work-item counters,
// sequence ranking, work lists, partial sums of a kv-split), held by every device the library is loaded on until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress: the device address it yields (one
// per device) is what kernels and copies are given.  Its size, HSTU_NOALLOC_SCRATCH_BYTES, is part of the interface.
static __device__ __align__(256) unsigned char scratch[HSTU_NOALLOC_SCRATCH_BYTES];

namespace hstu {

// Work done ahead of the forward kernel, in the caller's workspace (either part may be absent):
// * order[rank] = sequence index, longest sequence first (ties by index).  One wave per sequence: its lanes share
//   out the other sequences and count, by ballot, those that precede it.
// * queue[16 * xcd] = first work item the persistent workgroups of that XCD have not taken statically.
__global__ __launch_bounds__(256) void hstu_prep_kernel(const void* offsets, int offsets_i64, int B, int* order, int* queue,
                                                        int queue_start) {
    if (queue && blockIdx.x == 0 && threadIdx.x < 8) queue[threadIdx.x * 16] = queue_start;
    if (!order) return;
    auto len = [&](int j) -> long long {
        return offsets_i64 ? ((const long long*)offsets)[j + 1] - ((const long long*)offsets)[j]
                           : (long long)(((const int*)offsets)[j + 1] - ((const int*)offsets)[j]);
    };
    const int i = (blockIdx.x * 256 + threadIdx.x) >> 6;  // wave-uniform
    const int lane = threadIdx.x & 63;
    if (i >= B) return;
    const long long ni = len(i);
    int rank = 0;
    for (int j0 = 0; j0 < B; j0 += 64) {
        const int j = j0 + lane;
        bool before = false;
        if (j < B) {
            const long long nj = len(j);
            before = (nj > ni) || (nj == ni && j < i);
        }
        rank += __popcll(__ballot(before));
    }
    if (lane == 0) order[rank] = i;
}

// The caller contract checked on the device: report[0] = number of sequences that break it, report[1] = the first
// such sequence, report[2] = what it breaks (bit 0: offsets decrease, 1: longer than max_seq_len, 2: num_targets outside
// [0, length], 3: fewer non-target positions than contextual_seq_len, 4: shorter than delta_size), report[3] = 1 if
// seq_offsets[0] != 0 or seq_offsets[batch] != total_kv.  One thread per sequence.
__global__ __launch_bounds__(256) void hstu_check_contract_kernel(const void* offsets, int offsets_i64, const void* targets, int targets_i64,
                                                                   int B, long long total_kv, int max_seq_len, int c, int delta,
                                                                   int* report) {
    auto off = [&](int j) -> long long { return offsets_i64 ? ((const long long*)offsets)[j] : (long long)((const int*)offsets)[j]; };
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b == 0 && (off(0) != 0 || off(B) != total_kv)) report[3] = 1;
    if (b >= B) return;
    const long long n = off(b + 1) - off(b);
    long long t = 0;
    if (targets) t = targets_i64 ? ((const long long*)targets)[b] : (long long)((const int*)targets)[b];
    int what = 0;
    if (n < 0) what |= 1;
    if (n > max_seq_len) what |= 2;
    if (t < 0 || t > n) what |= 4;
    if (n > 0 && n - t < c) what |= 8;
    if (delta > 0 && n < delta) what |= 16;
    if (what) {
        atomicAdd(report, 1);
        atomicMin(report + 1, b);
        atomicOr(report + 2, what);
    }
}

}  // namespace hstu

namespace {

constexpr int kMaxSortBatch = 8192;  // beyond this the quadratic ranking is not worth its time

thread_local char g_last_error[256] = "";

void set_last_error(const char* what, hipError_t e) {
    snprintf(g_last_error, sizeof(g_last_error), "%s: %s", what, hipGetErrorString(e));
}

struct TileConfig {
    const char* name;
    int qt, nw, bn;  // query tiles (of 32 rows) per wave, waves per workgroup, kv rows per tile
};
// id 1..: see hstu_hip_tile_configs()
const TileConfig kConfigs[] = {
    {"m128n64w4", 1, 4, 64},
    {"m256n64w8pp", 1, 8, 64},
    {"m128n64w4pl", 1, 4, 64},
};
constexpr int kNumConfigs = sizeof(kConfigs) / sizeof(kConfigs[0]);

// `p` arrives complete (num_mb, pairs_per_xcd, slots_per_xcd, queue ...); these only pick the instantiation.
template <class TT, int DQK, int DV, int QT, int NW, int BN, int OCC>
int launch(const hstu::FwdParams& p, hipStream_t stream) {
    // + 64: with dv = 16 the transposing reads of the unused upper half of the tile reach past the last V row
    constexpr int smem = 2 * BN * (DQK + DV) * TT::ES + 64;
    auto kern = hstu::hstu_fwd_kernel<TT, DQK, DV, QT, NW, BN, OCC>;
    // once per device (the attribute belongs to the device's copy of the kernel); raising the dynamic LDS limit is
    // idempotent, so racing threads only set the same value twice
    static bool attr_done[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    if (dev < 0 || !attr_done[dev]) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) {
            set_last_error("hipFuncSetAttribute", e);
            return HSTU_ERR_LAUNCH;
        }
        if (dev >= 0) attr_done[dev] = true;
    }
    const long long grid = (long long)p.slots_per_xcd * 8;  // one workgroup per work item
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), smem, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_error("kernel launch", e);
        return HSTU_ERR_LAUNCH;
    }
    return HSTU_OK;
}

template <class TT, int DQK, int DV, int BN, int NG>
int launch_pp(const hstu::FwdParams& p, int grid_per_xcd, int64_t total_q, hipStream_t stream) {
    if constexpr (NG == 0) {  // the streaming form of the 8-wave kernel
        hipLaunchKernelGGL((hstu::hstu_fwd_stream_kernel<TT, DQK, DV, BN>), dim3((unsigned)grid_per_xcd * 8), dim3(512), 0, stream, p);
    } else {
        hipLaunchKernelGGL((hstu::hstu_fwd_pp_kernel<TT, DQK, DV, BN, NG>), dim3((unsigned)grid_per_xcd * 8), dim3(NG * 256), 0, stream,
                           p);  // LDS is a static array
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_error("kernel launch", e);
        return HSTU_ERR_LAUNCH;
    }
    if (p.kv_splits > 1) {
        const long long threads = (long long)total_q * p.H * (DV / 4);
        const long long blocks = (threads + 255) / 256;
        if (blocks > 0x7fffffffLL) return HSTU_ERR_BAD_SHAPE;
        hipLaunchKernelGGL(hstu::hstu_reduce_splits_kernel<typename TT::out_elem>, dim3((unsigned)blocks), dim3(256), 0, stream,
                           p, total_q, DV, NG == 1 ? 128 : 256);
        e = hipGetLastError();
        if (e != hipSuccess) {
            set_last_error("reduce kernel launch", e);
            return HSTU_ERR_LAUNCH;
        }
    }
    return HSTU_OK;
}

template <class TT, int D>
int launch_cfg(const hstu::FwdParams& p, int cfg, int grid_per_xcd, int64_t total_q, hipStream_t stream) {
    if (cfg == 2) return launch_pp<TT, D, D, 64, 0>(p, grid_per_xcd, total_q, stream);  // 8 waves, two groups: the streaming kernel
    if (cfg == 3) return launch_pp<TT, D, D, 64, 1>(p, grid_per_xcd, total_q, stream);  // 4 waves, one group
    return launch<TT, D, D, 1, 4, 64, 2>(p, stream);
}

// Unequal or 16-wide head dims: only the barrier-per-tile kernel is generic in (dqk, dv).
template <class TT, int DQK>
int launch_mixed_dv(const hstu::FwdParams& p, int dv, hipStream_t stream) {
    switch (dv) {
        case 16:
            if constexpr (TT::ES == 2) return launch<TT, DQK, 16, 1, 4, 64, 2>(p, stream);
            return HSTU_ERR_BAD_HEAD_DIM;
        case 32: return launch<TT, DQK, 32, 1, 4, 64, 2>(p, stream);
        case 64: return launch<TT, DQK, 64, 1, 4, 64, 2>(p, stream);
        case 128: return launch<TT, DQK, 128, 1, 4, 64, 2>(p, stream);
        default: return HSTU_ERR_BAD_HEAD_DIM;
    }
}

template <class TT>
int launch_mixed(const hstu::FwdParams& p, int dqk, int dv, hipStream_t stream) {
    switch (dqk) {
        case 16:
            if constexpr (TT::ES == 2) return launch_mixed_dv<TT, 16>(p, dv, stream);
            return HSTU_ERR_BAD_HEAD_DIM;
        case 32: return launch_mixed_dv<TT, 32>(p, dv, stream);
        case 64: return launch_mixed_dv<TT, 64>(p, dv, stream);
        case 128: return launch_mixed_dv<TT, 128>(p, dv, stream);
        default: return HSTU_ERR_BAD_HEAD_DIM;
    }
}

template <class TT>
int launch_dim(const hstu::FwdParams& p, int d, int dv, int cfg, int grid_per_xcd, int64_t total_q, hipStream_t stream) {
    if (cfg == 1 && (d != dv || d == 16)) return launch_mixed<TT>(p, d, dv, stream);
    switch (d) {
        case 32: return launch_cfg<TT, 32>(p, cfg, grid_per_xcd, total_q, stream);
        case 64: return launch_cfg<TT, 64>(p, cfg, grid_per_xcd, total_q, stream);
        case 128: return launch_cfg<TT, 128>(p, cfg, grid_per_xcd, total_q, stream);
        default: return HSTU_ERR_BAD_HEAD_DIM;
    }
}

// What a call will do, from sizes the host knows without reading the offsets.
struct Plan {
    int cfg;               // tile configuration, 1-based
    int splits;            // workgroups per row block along kv (1 = no split)
    int chunk;             // kv tiles per run when split
    // the workspace, in this order:
    size_t queue_bytes;    // work-item counters and list lengths of the persistent kernels
    size_t order_bytes;    // sequence ranking
    size_t counts_bytes;   // runs per row block of a kv-split
    size_t partial_bytes;  // fp32 partial outputs of the runs (256-byte aligned: 256 bytes of slack are added)
    size_t items_bytes;    // work lists: 8 lists of 32-byte records (see FwdParams::items)
    size_t cast_bytes;     // fp16 copies of fp32 q, k, v, each 256-byte aligned
    size_t total() const {
        return queue_bytes + order_bytes + counts_bytes + (partial_bytes ? partial_bytes + 256 : 0) + items_bytes + cast_bytes;
    }
};

constexpr int kMaxSplits = 8;
constexpr int kTileRows = 64;  // kv rows per tile of every configuration

// The pipelined kernels address the rows of a sequence through buffer descriptors with 32-bit byte offsets: the longest
// sequence times the largest row stride has to stay below 2^32 bytes.
bool rows_fit_buffer_offsets(const HstuFwdArgs* a) {
    const int64_t es = a->dtype == HSTU_FP8_E4M3 ? 1 : 2;
    int64_t rs = a->q_row_stride > a->k_row_stride ? a->q_row_stride : a->k_row_stride;
    if (a->v_row_stride > rs) rs = a->v_row_stride;
    return (int64_t)a->max_seq_len * rs * es < (1LL << 32);
}

Plan make_plan(const HstuFwdArgs* a) {
    Plan pl = {0, 1, 0, 0, 0, 0, 0, 0, 0};
    // The streaming two-group kernel (256-row blocks, one workgroup per CU) wins when the average sequence is long;
    // the one-group pipeline (128-row blocks, two workgroups per CU) wastes less on short or very uneven sequences
    // and in delta mode.
    pl.cfg = a->tile_config;
    const long long avg_tiles = a->batch > 0 ? a->total_kv / a->batch / kTileRows : 0;
    if (a->dqk != a->dv || a->dqk == 16) pl.cfg = 1;  // the only kernel generic in (dqk, dv)
    if (pl.cfg == 0 && !rows_fit_buffer_offsets(a)) pl.cfg = 1;  // the only kernel with 64-bit row addresses
    if (a->dtype == HSTU_FP32) {
        pl.cfg = 1;  // and the only one with an fp32 store
        pl.cast_bytes = 2 * ((size_t)a->total_q * a->heads * a->dqk + (size_t)a->total_kv * a->heads * (a->dqk + a->dv)) + 4 * 256;
    }
    if (pl.cfg == 0) {
        if (a->delta_size == 0) {
            // (measured, H = 4, d = 128, by average length: 544 rows -- the streaming kernel is 6 % behind; 900 to 1000
            // -- 1 to 3 % ahead; 1280 -- level; 1800 -- 3 % ahead; 2048 to 2560 -- 6 to 8 % ahead)
            pl.cfg = avg_tiles >= 960 / kTileRows ? 2 : 3;
        } else {
            // few long histories: 256-row blocks, whose kv range is then split below so that every CU gets one
            const long long blocks256 = (long long)a->batch * a->heads * ((a->delta_size + 255) / 256);
            pl.cfg = (blocks256 * 2 <= 256 && avg_tiles >= 32) ? 2 : 3;
        }
    }
    if (a->sort_by_length && a->batch >= 2 && a->batch <= kMaxSortBatch) pl.order_bytes = (size_t)a->batch * sizeof(int);
    if (pl.cfg < 2 || a->batch <= 0) return pl;
    pl.queue_bytes = 8 * 64 + 64;  // one counter per XCD, 64 bytes apart, then the 8 list lengths
    const int bm = pl.cfg == 2 ? 256 : 128;
    const int rows_per_pair = a->delta_size > 0 ? a->delta_size : a->max_seq_len;
    const long long blocks = (long long)a->batch * a->heads * ((rows_per_pair + bm - 1) / bm);
    const int max_tiles = (a->max_seq_len + kTileRows - 1) / kTileRows;
    int s = 1;
    if (a->kv_splits > 0) {
        s = a->kv_splits;
    } else if (a->delta_size > 0) {
        // Delta mode has few query rows per sequence: with a small batch the row blocks alone do not fill the
        // 256 CUs.  Cut the kv range so that the chip is just filled (more runs than that only add partial-sum
        // traffic: with every CU busy the clock drops and the time per tile rises), in runs of at least 16 tiles.
        const long long resident = pl.cfg == 2 ? 256 : 512;  // workgroups the chip holds at once
        long long want = resident / blocks;
        if (want > max_tiles / 16) want = max_tiles / 16;
        if (want > kMaxSplits) want = kMaxSplits;
        if (want >= 2) s = (int)want;
    }
    // Work lists for ragged batches (equal lengths are dealt arithmetically, a kv-split enumerates its runs
    // arithmetically too): 32 bytes per possible item; beyond 64 MB the arithmetic enumeration stays.
    const bool uniform = a->delta_size == 0 && a->total_kv == (int64_t)a->batch * a->max_seq_len;
    if (s == 1 && !uniform) {
        const unsigned long long bytes = (unsigned long long)((a->batch * (long long)a->heads + 7) / 8) * (unsigned long long)((rows_per_pair + bm - 1) / bm) * 256ull;
        if (bytes <= (64ull << 20)) pl.items_bytes = (size_t)bytes + 32;  // 32: room to align the records
    }
    if (s > 1) {
        pl.splits = s;
        pl.chunk = (max_tiles + s - 1) / s;
        pl.counts_bytes = (size_t)blocks * sizeof(int);
        pl.partial_bytes = (size_t)s * (size_t)a->total_q * a->heads * a->dv * sizeof(float);
    }
    return pl;
}

// Constants for fast_div (device side): x / d == (x * magic) >> (32 + shift) for 0 <= x < 2^31; magic 0 means d == 1.
void fast_div_constants(unsigned d, unsigned* magic, unsigned* shift) {
    if (d <= 1) {
        *magic = 0;
        *shift = 0;
        return;
    }
    unsigned l = 0;
    while ((1ull << l) < d) ++l;  // ceil(log2 d) >= 1
    *magic = (unsigned)((1ull << (31 + l)) / d + 1);
    *shift = l - 1;
}

void fill_decode_params(hstu::FwdParams& p) {
    hstu::DecodeParams& d = p.dec;
    memset(&d, 0, sizeof(d));
    d.items = p.items;
    d.nitems = p.nitems;
    d.order = p.order;
    d.offsets = p.offsets;
    d.targets = p.targets;
    d.items_cap = p.items_cap;
    d.kv_splits = p.kv_splits;
    d.kv_chunk = p.kv_chunk;
    d.c = p.c;
    d.pairs_per_xcd = p.pairs_per_xcd;
    d.num_mb = p.num_mb;
    d.B = p.B;
    d.H = p.H;
    d.uniform = p.uniform;
    d.max_seq_len = p.max_seq_len;
    d.offsets_i64 = p.offsets_i64;
    d.targets_i64 = p.targets_i64;
    d.delta = p.delta;
    d.w = p.w;
    d.f = p.f;
    d.mb_magic = p.mb_magic;
    d.mb_shift = p.mb_shift;
    d.h_magic = p.h_magic;
    d.h_shift = p.h_shift;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

// 1 if the current device is gfx950, 0 if not, cached per device ordinal (the kernels use gfx950-only
// instructions; the reference's native op makes the same kind of check, flash_common.cpp:420-422).
int current_device_is_gfx950() {
    static int cache[64];  // 0 unknown, 1 yes, 2 no; racing threads store the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (dev < 0 || dev >= 64) return 0;
    if (cache[dev] == 0) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
        cache[dev] = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
    }
    return cache[dev] == 1;
}

// Compute units of the current device (256 on MI355X), cached per device ordinal.
int current_device_cus() {
    static int cache[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cache[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cache[dev] = n;
    }
    return cache[dev];
}

}  // namespace

// for the library's other translation units; not exported
extern "C" __attribute__((visibility("hidden"))) int hstu_hip_device_is_gfx950(void) { return current_device_is_gfx950(); }
extern "C" __attribute__((visibility("hidden"))) void hstu_hip_set_last_error(const char* what, int hip_error) {
    set_last_error(what, (hipError_t)hip_error);
}

// order[rank] = sequence index, longest first, for the backward entry point's schedule; 0 or HSTU_ERR_LAUNCH
extern "C" __attribute__((visibility("hidden"))) int hstu_hip_launch_rank(const void* offsets, int offsets_i64, int batch, int* order,
                                                                          void* stream) {
    const unsigned blocks = (unsigned)(((long long)batch * 64 + 255) / 256);
    hipLaunchKernelGGL(hstu::hstu_prep_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, offsets, offsets_i64, batch, order,
                       (int*)nullptr, 0);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_error("rank kernel launch", e);
        return HSTU_ERR_LAUNCH;
    }
    return HSTU_OK;
}

extern "C" {

int hstu_hip_version(void) { return 101; }

const char* hstu_hip_status_string(int status) {
    switch (status) {
        case HSTU_OK: return "ok";
        case HSTU_ERR_NULL_POINTER: return "a required pointer is NULL";
        case HSTU_ERR_BAD_DTYPE: return "only bf16, fp16, fp8_e4m3 and fp32 data types are supported";
        case HSTU_ERR_BAD_HEAD_DIM: return "unsupported head dimension (built: dqk, dv in {16, 32, 64, 128}; 8-bit types from 32)";
        case HSTU_ERR_MISALIGNED:
            return "q/k/v/out must be 16-byte aligned with row and head strides that are multiples of 16 bytes";
        case HSTU_ERR_BAD_SHAPE: return "inconsistent sizes";
        case HSTU_ERR_UNSUPPORTED: return "argument combination not built";
        case HSTU_ERR_LAUNCH: return "HIP launch failed";
        case HSTU_ERR_BAD_DEVICE: return "current device is not gfx950";
        case HSTU_ERR_SCRATCH_LIMIT: return "the call needs more scratch memory than the library's fixed area holds";
        case HSTU_ERR_BUSY: return "the library's fixed scratch area is still in use by a call on another stream";
        default: return "unknown status";
    }
}

const char* hstu_hip_last_error(void) { return g_last_error; }

size_t hstu_hip_workspace_bytes(const HstuFwdArgs* a) {
    if (!a || a->batch <= 0 || a->heads <= 0 || a->total_q <= 0) return 0;
    return make_plan(a).total();
}

int hstu_hip_plan(const HstuFwdArgs* a, int32_t* tile_config, int32_t* kv_splits) {
    int rc = hstu_hip_check_args(a);
    if (rc != HSTU_OK) return rc;
    Plan pl = make_plan(a);
    if (pl.splits > 1 && !(a->workspace && (size_t)a->workspace_bytes >= pl.total()) && a->kv_splits <= 1) pl.splits = 1;
    if (tile_config) *tile_config = pl.cfg;
    if (kv_splits) *kv_splits = pl.splits;
    return HSTU_OK;
}

int hstu_hip_tile_configs(void) { return kNumConfigs; }

const char* hstu_hip_tile_config_name(int id) {
    if (id < 1 || id > kNumConfigs) return "";
    return kConfigs[id - 1].name;
}

int hstu_hip_check_args(const HstuFwdArgs* a) {
    if (!a) return HSTU_ERR_NULL_POINTER;
    if (a->dtype != HSTU_BF16 && a->dtype != HSTU_FP16 && a->dtype != HSTU_FP8_E4M3 && a->dtype != HSTU_FP32) return HSTU_ERR_BAD_DTYPE;
    if (a->batch < 0 || a->heads <= 0 || a->total_q < 0 || a->total_kv < 0 || a->max_seq_len <= 0 ||
        a->delta_size < 0 || a->max_attn_len < 0 || a->contextual_seq_len < 0 || a->min_full_attn_seq_len < 0)
        return HSTU_ERR_BAD_SHAPE;
    if (a->delta_size > 0 && a->total_q != (int64_t)a->batch * a->delta_size) return HSTU_ERR_BAD_SHAPE;
    if (a->delta_size == 0 && a->total_q != a->total_kv) return HSTU_ERR_BAD_SHAPE;
    if (a->total_kv > 0x7fffffffLL) return HSTU_ERR_BAD_SHAPE;
    if (a->tile_config < 0 || a->tile_config > kNumConfigs) return HSTU_ERR_BAD_SHAPE;
    if (a->kv_splits < 0 || a->kv_splits > kMaxSplits || (a->kv_splits > 1 && a->tile_config == 1)) return HSTU_ERR_BAD_SHAPE;
    if (a->workspace && (a->workspace_bytes < 0 || (reinterpret_cast<uintptr_t>(a->workspace) & 3) != 0)) return HSTU_ERR_MISALIGNED;
    if (a->attn_scale && (reinterpret_cast<uintptr_t>(a->attn_scale) & 3) != 0) return HSTU_ERR_MISALIGNED;
    if (a->attn_scale && a->delta_size > 0) return HSTU_ERR_UNSUPPORTED;  // the reference's cached form has no attn_scale
    // head dims 16 / 32 / 64 / 128, independently for q/k and v (the grid of the reference's tests,
    // hstu_attention_test.py:266-267; its native op wants them equal, flash_common.cpp:543-545); 8-bit rows are at
    // least 32 wide
    for (int d : {a->dqk, a->dv})
        if (d != 32 && d != 64 && d != 128 && !(d == 16 && a->dtype != HSTU_FP8_E4M3)) return HSTU_ERR_BAD_HEAD_DIM;
    // unequal or 16-wide dims and fp32 run on tile config 1 only
    if ((a->dqk != a->dv || a->dqk == 16 || a->dtype == HSTU_FP32) && a->tile_config > 1) return HSTU_ERR_UNSUPPORTED;
    // ... and so do sequences whose rows span 4 GB or more
    if (a->tile_config > 1 && !rows_fit_buffer_offsets(a)) return HSTU_ERR_UNSUPPORTED;
    if (a->total_q == 0 || a->batch == 0) return HSTU_OK;  // nothing to do; pointers may be anything
    if (!a->q || !a->k || !a->v || !a->out || !a->seq_offsets) return HSTU_ERR_NULL_POINTER;
    if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->out)) return HSTU_ERR_MISALIGNED;
    const int64_t strides[8] = {a->q_row_stride, a->q_head_stride, a->k_row_stride, a->k_head_stride,
                                a->v_row_stride, a->v_head_stride, a->o_row_stride, a->o_head_stride};
    // rows of q/k/v start on 16-byte boundaries: 8 elements of 16 bits, 16 of 8 bits, 4 of 32 bits; the output is 16
    // bit, or 32 bit for fp32 inputs
    const int64_t in_mask = a->dtype == HSTU_FP8_E4M3 ? 15 : a->dtype == HSTU_FP32 ? 3 : 7;
    const int64_t out_mask = a->dtype == HSTU_FP32 ? 3 : 7;
    for (int i = 0; i < 8; ++i)
        if (strides[i] < 0 || (strides[i] & (i < 6 ? in_mask : out_mask)) != 0) return HSTU_ERR_MISALIGNED;
    return HSTU_OK;
}

int hstu_hip_check_contract(const HstuFwdArgs* a, int32_t* report, void* stream_) {
    g_last_error[0] = 0;
    int rc = hstu_hip_check_args(a);
    if (rc != HSTU_OK) return rc;
    if (!report) return HSTU_ERR_NULL_POINTER;
    hipStream_t stream = (hipStream_t)stream_;
    // a small fill kernel would do as well; this copy is outside anything a caller captures (the check reads back).
    // The source outlives the call: an asynchronous copy from pageable memory may read it after this function returns.
    static const int32_t init[4] = {0, 0x7fffffff, 0, 0};
    hipError_t e = hipMemcpyAsync(report, init, sizeof(init), hipMemcpyHostToDevice, stream);
    if (e != hipSuccess) {
        set_last_error("hipMemcpyAsync", e);
        return HSTU_ERR_LAUNCH;
    }
    if (a->batch == 0 || !a->seq_offsets) return HSTU_OK;
    hipLaunchKernelGGL(hstu::hstu_check_contract_kernel, dim3((a->batch + 255) / 256), dim3(256), 0, stream, a->seq_offsets,
                       a->seq_offsets_i64, a->num_targets, a->num_targets_i64, a->batch, (long long)a->total_kv, a->max_seq_len,
                       a->contextual_seq_len, a->delta_size, report);
    e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_error("contract kernel launch", e);
        return HSTU_ERR_LAUNCH;
    }
    return HSTU_OK;
}

int hstu_hip_mha_fwd(const HstuFwdArgs* a, void* stream_) {
    g_last_error[0] = 0;
    int rc = hstu_hip_check_args(a);
    if (rc != HSTU_OK) return rc;
    if (a->total_q == 0 || a->batch == 0) return HSTU_OK;
    if (!current_device_is_gfx950()) return HSTU_ERR_BAD_DEVICE;
    hipStream_t stream = (hipStream_t)stream_;

    hstu::FwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = (const char*)a->q;
    p.k = (const char*)a->k;
    p.v = (const char*)a->v;
    p.o = (char*)a->out;
    p.q_rs = a->q_row_stride;
    p.q_hs = a->q_head_stride;
    p.k_rs = a->k_row_stride;
    p.k_hs = a->k_head_stride;
    p.v_rs = a->v_row_stride;
    p.v_hs = a->v_head_stride;
    p.o_rs = a->o_row_stride;
    p.o_hs = a->o_head_stride;
    p.offsets = a->seq_offsets;
    p.targets = a->num_targets;
    p.offsets_i64 = a->seq_offsets_i64;
    p.targets_i64 = a->num_targets_i64;
    p.B = a->batch;
    p.H = a->heads;
    p.max_seq_len = a->max_seq_len;
    p.delta = a->delta_size;
    p.w = a->max_attn_len;
    p.c = a->contextual_seq_len;
    p.f = a->min_full_attn_seq_len;
    p.c1 = -a->alpha * 1.4426950408889634f;
    p.oscale = a->alpha == 0.0f ? 0.0f : -1.0f / ((float)a->max_seq_len * 1.4426950408889634f);
    p.oscale_unit = a->alpha == 0.0f ? 0.0f : -1.0f / 1.4426950408889634f;
    p.attn_scale = (const float*)a->attn_scale;
    p.attn_scale_per_row = a->attn_scale_per_row;
    if (a->dtype == HSTU_FP8_E4M3) {
        // real value = stored value * scale: the score scales go into c1 (applied to the accumulator), the
        // value scale and the factor P is stored with go into the output scale
        p.c1 *= a->q_scale * a->k_scale;
        p.oscale *= a->v_scale / hstu::Fp8::PSCALE;
        p.oscale_unit *= a->v_scale / hstu::Fp8::PSCALE;
    }

    // Every use of the caller's scratch memory is an optimisation that never changes the result: without enough of
    // it an automatic choice falls back to the plain schedule, an explicit kv_splits > 1 is an error.
    Plan plan = make_plan(a);
    const bool ws_ok = a->workspace && (size_t)a->workspace_bytes >= plan.total();
    if (a->dtype == HSTU_FP32) {
        // the one use of the workspace that is not optional: rounded copies of the inputs
        if (!ws_ok) return a->workspace ? HSTU_ERR_BAD_SHAPE : HSTU_ERR_NULL_POINTER;
        char* cur = (char*)a->workspace + plan.total() - plan.cast_bytes;
        const void* src[3] = {a->q, a->k, a->v};
        const int64_t rs[3] = {a->q_row_stride, a->k_row_stride, a->v_row_stride};
        const int64_t hs[3] = {a->q_head_stride, a->k_head_stride, a->v_head_stride};
        const int64_t rows[3] = {a->total_q, a->total_kv, a->total_kv};
        const int d[3] = {a->dqk, a->dqk, a->dv};
        const char** dst[3] = {&p.q, &p.k, &p.v};
        int64_t* prs[3] = {&p.q_rs, &p.k_rs, &p.v_rs};
        int64_t* phs[3] = {&p.q_hs, &p.k_hs, &p.v_hs};
        for (int i = 0; i < 3; ++i) {
            cur = (char*)((reinterpret_cast<uintptr_t>(cur) + 255) & ~(uintptr_t)255);
            const long long threads = (long long)rows[i] * a->heads * (d[i] / 8);
            const long long blocks = (threads + 255) / 256;
            if (blocks > 0x7fffffffLL) return HSTU_ERR_BAD_SHAPE;
            if (blocks > 0) {
                hipLaunchKernelGGL(hstu::hstu_cast_f32_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const float*)src[i],
                                   rs[i], hs[i], rows[i], a->heads, d[i], (_Float16*)cur);
                hipError_t e = hipGetLastError();
                if (e != hipSuccess) {
                    set_last_error("cast kernel launch", e);
                    return HSTU_ERR_LAUNCH;
                }
            }
            *dst[i] = cur;
            *prs[i] = (int64_t)a->heads * d[i];
            *phs[i] = d[i];
            cur += (size_t)rows[i] * a->heads * d[i] * 2;
        }
    }
    if (plan.splits > 1 && !ws_ok) {
        if (a->kv_splits > 1) return a->workspace ? HSTU_ERR_BAD_SHAPE : HSTU_ERR_NULL_POINTER;
        plan.splits = 1;
        plan.partial_bytes = plan.counts_bytes = 0;
    }
    char* ws = (char*)a->workspace;
    const size_t ws_bytes = a->workspace ? (size_t)a->workspace_bytes : 0;
    int* queue = plan.queue_bytes > 0 && ws_bytes >= plan.queue_bytes ? (int*)ws : nullptr;
    int* order = plan.order_bytes > 0 && ws_bytes >= plan.queue_bytes + plan.order_bytes ? (int*)(ws + plan.queue_bytes) : nullptr;
    if (plan.splits > 1) {
        char* base = ws + plan.queue_bytes + plan.order_bytes;
        p.split_counts = (int*)base;
        p.partial = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(base + plan.counts_bytes) + 255) & ~(uintptr_t)255);
        p.partial_stride = (int64_t)a->total_q * a->heads * a->dv;
        p.kv_chunk = plan.chunk;
    }
    p.kv_splits = plan.splits;

    // the grid: work items per XCD, and for the persistent kernels the workgroups that stay resident (one 8-wave
    // or two 4-wave workgroups per CU; the same number on every XCD)
    const int cfg = plan.cfg;
    const int rows_per_pair = a->delta_size > 0 ? a->delta_size : a->max_seq_len;
    const long long num_pairs = (long long)a->batch * a->heads;
    const int bm = cfg == 2 ? 256 : 128;
    p.num_mb = (rows_per_pair + bm - 1) / bm;
    const long long pairs_per_xcd = (num_pairs + 7) / 8;
    const long long slots = pairs_per_xcd * p.num_mb * plan.splits;
    if (slots <= 0) return HSTU_OK;
    if (slots * 8 > 0x7fffffffLL) return HSTU_ERR_BAD_SHAPE;
    p.pairs_per_xcd = (int)pairs_per_xcd;
    p.slots_per_xcd = (int)slots;
    fast_div_constants((unsigned)p.num_mb, &p.mb_magic, &p.mb_shift);
    fast_div_constants((unsigned)p.H, &p.h_magic, &p.h_shift);
    long long resident = (long long)current_device_cus() * (cfg == 2 ? 1 : 2) / 8;
    if (resident < 1) resident = 1;
    const int grid_per_xcd = (int)(slots < resident ? slots : resident);
    if (cfg < 2 || slots <= grid_per_xcd) queue = nullptr;  // every workgroup has exactly one item
    int* items = nullptr;
    if (queue && plan.items_bytes > 0 && ws_bytes >= plan.total()) items = (int*)(ws + plan.total() - plan.cast_bytes - plan.items_bytes);
    // Equal-length sequences (every one as long as max_seq_len allows): dealing the items with a fixed stride is
    // perfectly balanced and keeps all workgroups of an XCD on the same (sequence, head) pair at the same time,
    // which measures 4-5 % faster than the counter; any other batch needs the counter for balance.
    if (a->delta_size == 0 && a->total_kv == (int64_t)a->batch * a->max_seq_len) {
        queue = nullptr;
        // ... and (the caller's contract: no sequence is longer than max_seq_len) sequence b is rows b * max_seq_len
        // onwards: the kernels need neither the offsets nor a ranking by length
        p.uniform = 1;
        order = nullptr;
    }

    // ahead of the forward kernel: sequence ranking and / or the start value of the work-item counters
    if (order || queue) {
        const int blocks = order ? (a->batch + 3) / 4 : 1;
        hipLaunchKernelGGL(hstu::hstu_prep_kernel, dim3(blocks), dim3(256), 0, stream, a->seq_offsets, a->seq_offsets_i64,
                           a->batch, order, queue, grid_per_xcd);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            set_last_error("prep kernel launch", e);
            return HSTU_ERR_LAUNCH;
        }
    }
    p.order = order;
    p.queue = queue;
    if (items && queue) {
        // the lists are 32-byte records behind everything else in the workspace; align them
        items = (int*)((reinterpret_cast<uintptr_t>(items) + 31) & ~(uintptr_t)31);
        p.items_cap = (int)slots;
        hipLaunchKernelGGL(hstu::hstu_plan_kernel, dim3(8), dim3(HSTU_PLAN_THREADS), 0, stream, p, bm, 64, queue + 8 * 16, items);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            set_last_error("plan kernel launch", e);
            return HSTU_ERR_LAUNCH;
        }
        p.items = items;
        p.nitems = queue + 8 * 16;
    }

    // (after everything above: the block decode_work reads is made of copies)
    fill_decode_params(p);
    if (a->dtype == HSTU_FP32) return launch_mixed<hstu::Fp16F32>(p, a->dqk, a->dv, stream);
    if (a->dtype == HSTU_BF16) return launch_dim<hstu::Bf16>(p, a->dqk, a->dv, cfg, grid_per_xcd, a->total_q, stream);
    if (a->dtype == HSTU_FP16) return launch_dim<hstu::Fp16>(p, a->dqk, a->dv, cfg, grid_per_xcd, a->total_q, stream);
    return launch_dim<hstu::Fp8>(p, a->dqk, a->dv, cfg, grid_per_xcd, a->total_q, stream);
}

namespace {

// Per device, set up on the first call with that device current: the device address of `scratch` (each device holds
// its own copy of the array at its own address) and an event that marks the end of the last call that used the area.
struct NoallocState {
    void* scratch = nullptr;
    hipEvent_t done = nullptr;
    hipStream_t last_stream = nullptr;
    bool in_use = false;  // `done` has been recorded
};
std::mutex g_noalloc_mutex;

NoallocState* noalloc_state_of_current_device() {
    static NoallocState state[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    NoallocState& st = state[dev];
    if (!st.scratch) {
        void* ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            set_last_error("hipGetSymbolAddress(scratch)", e);
            return nullptr;
        }
        e = hipEventCreateWithFlags(&st.done, hipEventDisableTiming);
        if (e != hipSuccess) {
            set_last_error("hipEventCreateWithFlags", e);
            return nullptr;
        }
        st.scratch = ptr;
    }
    return &st;
}

}  // namespace

int hstu_hip_mha_fwd_noalloc(const HstuFwdArgs* a, void* stream_) {
    g_last_error[0] = 0;
    int rc = hstu_hip_check_args(a);
    if (rc != HSTU_OK) return rc;
    if (a->total_q == 0 || a->batch == 0) return HSTU_OK;
    if (!current_device_is_gfx950()) return HSTU_ERR_BAD_DEVICE;
    const size_t need = make_plan(a).total();
    if (need > (size_t)HSTU_NOALLOC_SCRATCH_BYTES) {
        snprintf(g_last_error, sizeof(g_last_error), "this call would use %zu bytes of scratch memory; the fixed area holds %zu", need,
                 (size_t)HSTU_NOALLOC_SCRATCH_BYTES);
        return HSTU_ERR_SCRATCH_LIMIT;
    }
    hipStream_t stream = (hipStream_t)stream_;
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);  // check, launch and record belong together
    NoallocState* st = noalloc_state_of_current_device();
    if (!st) return HSTU_ERR_LAUNCH;
    // A call on another stream while the last one has not finished would race on the area.  (Not under capture: an
    // event recorded into a graph cannot be queried, and a captured launch runs whenever the graph is replayed.)
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(stream, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
    if (!capturing && st->in_use && st->last_stream != stream && hipEventQuery(st->done) == hipErrorNotReady) {
        snprintf(g_last_error, sizeof(g_last_error), "the scratch area of this device is in use by a call on another stream");
        return HSTU_ERR_BUSY;
    }
    HstuFwdArgs b = *a;
    b.workspace = st->scratch;  // the device address, never the array's name
    b.workspace_bytes = (int64_t)HSTU_NOALLOC_SCRATCH_BYTES;
    // Everything the kernels read from the area is written earlier in the same call (counters and ranking by the prep
    // kernel, work lists by the plan kernel, run counts and partial sums by the forward kernel), so what an earlier
    // call left behind is never looked at and nothing has to be cleared.
    rc = hstu_hip_mha_fwd(&b, stream_);
    if (rc == HSTU_OK && !capturing && hipEventRecord(st->done, stream) == hipSuccess) {
        st->last_stream = stream;
        st->in_use = true;
    }
    return rc;
}

}  // extern "C"

namespace {

// Largest power of two <= 16 that divides every value given (addresses, strides, row size).
int common_vector_bytes(std::initializer_list<uint64_t> values) {
    uint64_t all = 16;
    for (uint64_t v : values) all |= v;
    int vec = 1;
    while (vec < 16 && (all & vec) == 0) vec <<= 1;
    return vec;
}

constexpr int kJaggedRows = 32;  // joined rows per workgroup

int check_jagged_args(const HstuJaggedCopyArgs* a) {
    if (!a) return HSTU_ERR_NULL_POINTER;
    if (a->batch < 0 || a->row_bytes < 0 || a->max_len_left < 0 || a->max_len_right < 0 || a->total_left < 0 || a->total_right < 0)
        return HSTU_ERR_BAD_SHAPE;
    if (a->left_row_stride < a->row_bytes || a->right_row_stride < a->row_bytes || a->joined_row_stride < a->row_bytes)
        return HSTU_ERR_BAD_SHAPE;
    if (!a->offsets_left && a->total_left != (int64_t)a->batch * a->max_len_left) return HSTU_ERR_BAD_SHAPE;
    if (!a->offsets_right && a->total_right != (int64_t)a->batch * a->max_len_right) return HSTU_ERR_BAD_SHAPE;
    if (a->batch == 0 || a->row_bytes == 0 || a->total_left + a->total_right == 0) return HSTU_OK;
    if (!a->joined || (a->total_left > 0 && !a->left) || (a->total_right > 0 && !a->right)) return HSTU_ERR_NULL_POINTER;
    return HSTU_OK;
}

template <bool SPLIT>
int launch_jagged_copy(const HstuJaggedCopyArgs* a, hipStream_t stream) {
    g_last_error[0] = 0;
    int rc = check_jagged_args(a);
    if (rc != HSTU_OK) return rc;
    if (a->batch == 0 || a->row_bytes == 0 || a->total_left + a->total_right == 0) return HSTU_OK;
    hstu::JaggedCopyParams p;
    p.left = (char*)a->left;
    p.right = (char*)a->right;
    p.joined = (char*)a->joined;
    p.left_rs = a->left_row_stride;
    p.right_rs = a->right_row_stride;
    p.joined_rs = a->joined_row_stride;
    p.row_bytes = a->row_bytes;
    p.offsets_left = a->offsets_left;
    p.offsets_right = a->offsets_right;
    p.offsets_left_i64 = a->offsets_left_i64;
    p.offsets_right_i64 = a->offsets_right_i64;
    p.batch = a->batch;
    p.max_len_left = a->max_len_left;
    p.max_len_right = a->max_len_right;
    const long long rows = (long long)a->max_len_left + a->max_len_right;
    const long long gx = (rows + kJaggedRows - 1) / kJaggedRows;
    if (gx <= 0) return HSTU_OK;
    if (gx > 0x7fffffffLL || a->batch > 65535) return HSTU_ERR_BAD_SHAPE;  // grid.y limit
    const dim3 grid((unsigned)gx, (unsigned)a->batch);
    const int vec = common_vector_bytes({(uint64_t)(uintptr_t)a->left, (uint64_t)(uintptr_t)a->right, (uint64_t)(uintptr_t)a->joined,
                                         (uint64_t)a->left_row_stride, (uint64_t)a->right_row_stride,
                                         (uint64_t)a->joined_row_stride, (uint64_t)a->row_bytes});
    switch (vec) {
        case 16: hipLaunchKernelGGL((hstu::hstu_jagged_copy_kernel<SPLIT, 16, kJaggedRows>), grid, dim3(256), 0, stream, p); break;
        case 8: hipLaunchKernelGGL((hstu::hstu_jagged_copy_kernel<SPLIT, 8, kJaggedRows>), grid, dim3(256), 0, stream, p); break;
        case 4: hipLaunchKernelGGL((hstu::hstu_jagged_copy_kernel<SPLIT, 4, kJaggedRows>), grid, dim3(256), 0, stream, p); break;
        case 2: hipLaunchKernelGGL((hstu::hstu_jagged_copy_kernel<SPLIT, 2, kJaggedRows>), grid, dim3(256), 0, stream, p); break;
        default: hipLaunchKernelGGL((hstu::hstu_jagged_copy_kernel<SPLIT, 1, kJaggedRows>), grid, dim3(256), 0, stream, p); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_error("jagged copy kernel launch", e);
        return HSTU_ERR_LAUNCH;
    }
    return HSTU_OK;
}

}  // namespace

extern "C" {

int hstu_hip_concat_2d_jagged(const HstuJaggedCopyArgs* a, void* stream) { return launch_jagged_copy<false>(a, (hipStream_t)stream); }

int hstu_hip_split_2d_jagged(const HstuJaggedCopyArgs* a, void* stream) { return launch_jagged_copy<true>(a, (hipStream_t)stream); }

int hstu_hip_jagged_write_tail(void* joined, int64_t joined_row_stride, const void* offsets, int32_t offsets_i64, const void* tail,
                               int64_t tail_row_stride, int64_t row_bytes, int32_t batch, int32_t tail_len, void* stream_) {
    g_last_error[0] = 0;
    if (batch < 0 || tail_len < 0 || row_bytes < 0 || joined_row_stride < row_bytes || tail_row_stride < row_bytes) return HSTU_ERR_BAD_SHAPE;
    if (batch == 0 || tail_len == 0 || row_bytes == 0) return HSTU_OK;
    if (!joined || !offsets || !tail) return HSTU_ERR_NULL_POINTER;
    if (batch > 65535) return HSTU_ERR_BAD_SHAPE;
    const dim3 grid((unsigned)((tail_len + kJaggedRows - 1) / kJaggedRows), (unsigned)batch);
    hipStream_t stream = (hipStream_t)stream_;
    const int vec = common_vector_bytes({(uint64_t)(uintptr_t)joined, (uint64_t)(uintptr_t)tail, (uint64_t)joined_row_stride,
                                         (uint64_t)tail_row_stride, (uint64_t)row_bytes});
#define HSTU_TAIL_LAUNCH(V)                                                                                                   \
    hipLaunchKernelGGL((hstu::hstu_jagged_write_tail_kernel<V, kJaggedRows>), grid, dim3(256), 0, stream, (char*)joined,        \
                       joined_row_stride, offsets, offsets_i64, (const char*)tail, tail_row_stride, row_bytes, tail_len)
    switch (vec) {
        case 16: HSTU_TAIL_LAUNCH(16); break;
        case 8: HSTU_TAIL_LAUNCH(8); break;
        case 4: HSTU_TAIL_LAUNCH(4); break;
        case 2: HSTU_TAIL_LAUNCH(2); break;
        default: HSTU_TAIL_LAUNCH(1); break;
    }
#undef HSTU_TAIL_LAUNCH
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_last_error("jagged write-tail kernel launch", e);
        return HSTU_ERR_LAUNCH;
    }
    return HSTU_OK;
}

}  // extern "C"
