// Fused consumer of the attention output for gfx950: norm(attn) * act(u), the optional copies of u and attn beside it,
// the output projection and the residual in one kernel -- `joined` never exists in memory.
//
//     out[r, :] = x[r, :] + [u' | attn | y][r, :] @ W,     y = act(u) * norm(attn)
// (hstu_compute_output of the reference, ops/hstu_compute.py:107-214, in its forward, dropout-free form
// ops/pytorch/pt_hstu_linear.py:24-124; which blocks exist and what u' is: see HstuOutputArgs.)
//
// A workgroup of 8 waves owns 128 rows and all 512 output columns: wave (rh, cb) accumulates rows rh*64 .. +64 times
// columns cb*128 .. +128 (2 x 4 MFMA blocks of 32 x 32, 128 accumulator registers).  The depth K = blocks * d is
// walked in tiles of 32.  Per tile
//   * W[32 k, 512 n] (32 KB) is copied HBM/L2 -> LDS with global_load_lds_dwordx4 two tiles ahead (three slots), laid
//     out as four slabs of 128 columns in the format of the q/k/v producer (256-byte rows, chunk swizzle swz_w) and
//     read transposed (ds_read_b64_tr_b16) as the A operand of  C^T[n, r] += W^T[n, k] . joined^T[k, r];
//   * the 128 x 32 slice of `joined` (8 KB) is MADE by the workgroup: every thread loads 8 elements of attn and of u
//     one tile ahead, turns them into 8 elements of u', attn or y (statistics of the row from a pass over the
//     workgroup's attn rows at the start, kept in LDS) and writes them to one of three LDS slots, from where the waves
//     read their B operands (ds_read_b128, lane = row).
// One barrier per tile.  The epilogue turns the fp32 accumulators around in LDS (the W ring is dead by then), adds the
// residual row-contiguously in fp32, rounds once and stores whole 128-byte lines.
// HBM traffic: attn, u, x read once (u and attn again from L2 for their copies), out written once; W (K x 512, at most
// 3 MB) stays in every XCD's L2.
#pragma once
#include "hstu_common.h"
#include "hstu_uqvk_kernel.h"

namespace hstu {

struct OutputFusedParams {
    const char* attn;
    const char* u;
    const char* x;
    int64_t attn_rs, u_rs, x_rs;  // elements
    const char* norm_weight;
    const char* norm_bias;
    float eps;
    const char* w;  // [K, 512] row-major
    char* out;      // [rows, 512] dense
    int64_t rows;
    int d;           // heads * linear_dim: multiple of 32, at most 1024
    int heads;       // group norm: at most 8
    int group_lanes; // group norm: linear_dim / 8 (a power of two, at least 4); 0 = layer norm
    int blk_u, blk_x;  // 1: the copy of u (first) / of attn (before y) is part of `joined`
    int silu_u;      // layer norm: the copied u goes through SiLU; group norm: u does before both uses
    int mul_act;     // layer norm: 0 none, 1 sigmoid, 2 SiLU on the u that multiplies
};

constexpr int kOutWaves = 8, kOutRows = 128, kOutCols = 512, kOutTileK = 32;
constexpr int kOutWSlot = kOutTileK * kOutCols * 2;  // 32 KB
constexpr int kOutASlot = kOutRows * kOutTileK * 2;  // 8 KB
constexpr int kOutMaxHeads = 8;
constexpr int kOutStats = kOutRows * kOutMaxHeads * 8;
constexpr int kOutLds = 3 * kOutWSlot + 3 * kOutASlot + kOutStats;
constexpr int kOutStageRow = 64 * 4 + 16;  // staging row: 64 fp32 outputs + pad

__device__ __forceinline__ float out_sigmoid(float v) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v)); }

template <class TT, bool GROUP>
__global__ __launch_bounds__(kOutWaves * 64, 2) void hstu_output_fused_kernel(const OutputFusedParams p) {
    typedef typename TT::vec8 vec8;
    typedef typename TT::elem elem;
    constexpr int NPW = (kOutWSlot / 1024) / kOutWaves;  // W copy instructions per wave and tile: 4
    constexpr int PD = 3;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    char* const a_ring = smem + 3 * kOutWSlot;
    float* const stats = (float*)(smem + 3 * kOutWSlot + 3 * kOutASlot);  // [row][head] -> (mean, rstd)

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5, l32 = lane & 31;
    const int rh = wave >> 2, cb = wave & 3;
    const int64_t row0 = (int64_t)blockIdx.x * kOutRows;
    const int tpb = p.d / kOutTileK;             // tiles per block of `joined`
    const int nblocks = p.blk_u + p.blk_x + 1;
    const int ntiles = nblocks * tpb;

    // ---- W copies: instruction i of this wave moves chunks (wave + 8 i) * 64 + lane of the tile (slab, k row, chunk)
    unsigned coff[NPW];
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
        const int pidx = (wave + kOutWaves * i) * 64 + lane;
        const int slab = pidx >> 9, row = (pidx >> 4) & 31;
        const int logical = (pidx & 15) ^ swz_w(row);
        coff[i] = (unsigned)row * (unsigned)(kOutCols * 2) + slab * 256 + logical * 16;
    }
    auto issue_w = [&](int t) {
        char* slot = smem + (t % 3) * kOutWSlot;
        const char* src = p.w + (int64_t)t * kOutTileK * kOutCols * 2;
#pragma unroll
        for (int i = 0; i < NPW; ++i) global_load_lds16_soff(src, coff[i], slot + (wave + kOutWaves * i) * 1024);
    };
    issue_w(0);
    if (ntiles > 1) issue_w(1);

    // ---- statistics of this workgroup's attn rows: wave w takes rows 16 w .. +16, a lane chunks lane and lane + 64
    {
        const int chunks = p.d >> 3;
        for (int i = 0; i < 16; ++i) {
            const int lr = wave * 16 + i;
            int64_t r = row0 + lr;
            r = r < p.rows ? r : p.rows - 1;
            float v[2][8];
            float sum[2] = {0.f, 0.f};
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2) {
                const int c = lane + 64 * c2;
                if (c < chunks) {
                    const vec8 raw = *(const vec8*)(p.attn + (r * p.attn_rs + (int64_t)c * 8) * 2);
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        v[c2][j] = (float)raw[j];
                        sum[c2] += v[c2][j];
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[c2][j] = 0.f;
                }
            }
            if constexpr (GROUP) {
                const float inv_n = 1.0f / (float)(p.group_lanes * 8);
#pragma unroll
                for (int c2 = 0; c2 < 2; ++c2) {
                    const int c = lane + 64 * c2;
                    float s1 = sum[c2];
                    for (int dd = 1; dd < p.group_lanes; dd <<= 1) s1 += __shfl_xor(s1, dd, 64);
                    const float mean = s1 * inv_n;
                    float sq = 0.f;
                    if (c < chunks)
#pragma unroll
                        for (int j = 0; j < 8; ++j) sq += (v[c2][j] - mean) * (v[c2][j] - mean);
                    for (int dd = 1; dd < p.group_lanes; dd <<= 1) sq += __shfl_xor(sq, dd, 64);
                    if (c < chunks && (c & (p.group_lanes - 1)) == 0) {
                        const int head = c / p.group_lanes;
                        stats[(lr * kOutMaxHeads + head) * 2] = mean;
                        stats[(lr * kOutMaxHeads + head) * 2 + 1] = __builtin_amdgcn_rsqf(sq * inv_n + p.eps);
                    }
                }
            } else {
                const float inv_n = 1.0f / (float)p.d;
                float s1 = sum[0] + sum[1];
#pragma unroll
                for (int dd = 32; dd >= 1; dd >>= 1) s1 += __shfl_xor(s1, dd, 64);
                const float mean = s1 * inv_n;
                float sq = 0.f;
#pragma unroll
                for (int c2 = 0; c2 < 2; ++c2)
                    if (lane + 64 * c2 < chunks)
#pragma unroll
                        for (int j = 0; j < 8; ++j) sq += (v[c2][j] - mean) * (v[c2][j] - mean);
#pragma unroll
                for (int dd = 32; dd >= 1; dd >>= 1) sq += __shfl_xor(sq, dd, 64);
                if (lane == 0) {
                    stats[lr * kOutMaxHeads * 2] = mean;
                    stats[lr * kOutMaxHeads * 2 + 1] = __builtin_amdgcn_rsqf(sq * inv_n + p.eps);
                }
            }
        }
    }

    // ---- the slice of `joined` a thread makes per tile: row tid / 4, eight columns (tid % 4) * 8 .. of the tile
    const int arow = tid >> 2, achunk = tid & 3;
    int64_t arow_g = row0 + arow;
    arow_g = arow_g < p.rows ? arow_g : p.rows - 1;  // rows past the end repeat the last one; they are never stored
    const char* attn_row = p.attn + arow_g * p.attn_rs * 2 + achunk * 16;
    const char* u_row = p.u + arow_g * p.u_rs * 2 + achunk * 16;
    char* const a_dst = a_ring + arow * 64 + ((achunk ^ ((arow >> 2) & 3)) * 16);
    vec8 raw_a, raw_u;
    auto load_raw = [&](int t) __attribute__((always_inline)) {
        const int col = (t % tpb) * kOutTileK;
        raw_a = *(const vec8*)(attn_row + col * 2);
        raw_u = *(const vec8*)(u_row + col * 2);
    };
    auto make_a = [&](int t) __attribute__((always_inline)) {
        const int b = t / tpb;
        const int col = (t - b * tpb) * kOutTileK + achunk * 8;
        vec8 o;
        if (p.blk_u && b == 0) {  // u' : the copy of u
            o = raw_u;
            if (p.silu_u) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float uf = (float)raw_u[j];
                    o[j] = (elem)(uf * out_sigmoid(uf));
                }
            }
        } else if (p.blk_x && b == p.blk_u) {  // the copy of attn
            o = raw_a;
        } else {  // y
            const int head = GROUP ? col / (p.group_lanes * 8) : 0;
            const float mean = stats[(arow * kOutMaxHeads + head) * 2], rstd = stats[(arow * kOutMaxHeads + head) * 2 + 1];
            float wv[8], bv[8];
            if constexpr (GROUP) {
                const float w1 = (float)((const elem*)p.norm_weight)[head], b1 = (float)((const elem*)p.norm_bias)[head];
#pragma unroll
                for (int j = 0; j < 8; ++j) wv[j] = w1, bv[j] = b1;
            } else {
                const vec8 w8 = *(const vec8*)(p.norm_weight + col * 2), b8 = *(const vec8*)(p.norm_bias + col * 2);
#pragma unroll
                for (int j = 0; j < 8; ++j) wv[j] = (float)w8[j], bv[j] = (float)b8[j];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float uf = (float)raw_u[j];
                float mul = uf;
                if constexpr (GROUP) {
                    if (p.silu_u) mul = uf * out_sigmoid(uf);
                } else {
                    if (p.mul_act == 1) mul = out_sigmoid(uf);
                    if (p.mul_act == 2) mul = uf * out_sigmoid(uf);
                }
                o[j] = (elem)(mul * (((float)raw_a[j] - mean) * rstd * wv[j] + bv[j]));
            }
        }
        *HSTU_LDS(vec8, a_dst + (t % 3) * kOutASlot) = o;
    };
    load_raw(0);
    __syncthreads();  // the statistics are there
    make_a(0);
    if (ntiles > 1) load_raw(1);

    // ---- operand addresses
    int waddr[2][4];  // transposing reads of a W slab: lane supplies the address of 4 consecutive n of k row 8g + 4sec + j
    {
        const int i16 = lane & 15, half = (lane >> 4) & 1, jrow = i16 >> 2, q4 = i16 & 3;
#pragma unroll
        for (int sec = 0; sec < 2; ++sec) {
            const int row = 8 * g + 4 * sec + jrow;  // + 16 ks
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                const int chunk = dt * 4 + 2 * half + (q4 >> 1);
                waddr[sec][dt] = cb * (32 * 256) + row * 256 + ((chunk ^ swz_w(row)) * 16) + (q4 & 1) * 8;
            }
        }
    }
    int baddr[2][2];  // B operands: row rh*64 + rb*32 + l32 of the slice, columns 16 ks + 8 g .. +8
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int row = rh * 64 + rb * 32 + l32;
            baddr[rb][ks] = row * 64 + (((ks * 2 + g) ^ ((row >> 2) & 3)) * 16);
        }

    f32x16_t acc[2][4];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rb][dt][r] = 0.f;

    for (int t = 0; t < ntiles; ++t) {
        // W(t) has landed for this wave (what may still be in flight was issued after it: the copies of W(t+1) and the
        // loads for slice t+1), this thread's part of slice t is written ...
        if (t + 1 >= ntiles) __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0070 | (NPW + 2));
        __syncthreads();  // ... and so for every wave; nobody reads tile t - 1 any more, whose slots tile t + 2 takes
        // slice t + 1 first: its loads were the last thing issued a tile ago, so waiting for them waits for nothing newer
        if (t + 1 < ntiles) make_a(t + 1);
        if (t + 2 < ntiles) issue_w(t + 2);
        if (t + 2 < ntiles) load_raw(t + 2);
        const char* wt = smem + (t % 3) * kOutWSlot;
        const char* at = a_ring + (t % 3) * kOutASlot;
        vec8 breg[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) breg[rb][ks] = *HSTU_LDS(const vec8, at + baddr[rb][ks]);
        // 8 A operands (ks, dt) = (m / 4, m % 4), each used for the wave's two row blocks, requested PD ahead
        auto load_op = [&](int m) __attribute__((always_inline)) -> vec8 {
            const char* b = wt + (m >> 2) * 16 * 256;
            return read_vt_operand<TT>(b + waddr[0][m & 3], b + waddr[1][m & 3]);
        };
        vec8 fr[PD];
#pragma unroll
        for (int m = 0; m < PD; ++m) fr[m] = load_op(m);
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) acc[rb][m & 3] = TT::mfma(fr[m % PD], breg[rb][m >> 2], acc[rb][m & 3]);
            if (m + PD < 8) fr[m % PD] = load_op(m + PD);
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue: fp32 accumulators through this wave's staging area (the W ring is dead), + x, rounding, stores
    __syncthreads();
    char* stage = smem + wave * 32 * kOutStageRow;
    const int chunk = lane & 7, rsub = lane >> 3;  // 8 lanes cover one row's 64 columns, 8 rows per instruction
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
            for (int d2 = 0; d2 < 2; ++d2)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    f32x4_t o4;
#pragma unroll
                    for (int i = 0; i < 4; ++i) o4[i] = acc[rb][hf * 2 + d2][r4 * 4 + i];
                    *HSTU_LDS(f32x4_t, stage + l32 * kOutStageRow + (d2 * 32 + r4 * 8 + g * 4) * 4) = o4;
                }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = i * 8 + rsub;
                const int64_t r = row0 + rh * 64 + rb * 32 + row;
                const f32x4_t lo = *HSTU_LDS(const f32x4_t, stage + row * kOutStageRow + chunk * 32);
                const f32x4_t hi = *HSTU_LDS(const f32x4_t, stage + row * kOutStageRow + chunk * 32 + 16);
                if (r < p.rows) {
                    const int col = cb * 128 + hf * 64 + chunk * 8;
                    const vec8 xr = *(const vec8*)(p.x + (r * p.x_rs + col) * 2);
                    vec8 o;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        o[j] = (elem)(lo[j] + (float)xr[j]);
                        o[4 + j] = (elem)(hi[j] + (float)xr[4 + j]);
                    }
                    *(vec8*)(p.out + (r * kOutCols + col) * 2) = o;
                }
            }
        }
}

}  // namespace hstu
