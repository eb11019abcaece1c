// Fused producer of q, k, v for gfx950: layer norm + projection + bias + SiLU(u) in one kernel.
//
//     out[r, n] = act( sum_k LN(x)[r, k] * W[k, n] + bias[n] ),   act = SiLU for n < n_silu, identity otherwise
// (hstu_compute_uqvk of the reference, ops/hstu_compute.py:54-104; LN with fp32 statistics and its result rounded to the
// input type, ops/pytorch/pt_layer_norm.py:24-39).
//
// The depth of this product (d_model, at most 512) is small enough for a wave to keep its 32 normalised rows in
// registers for the whole kernel: they are the B operand of every MFMA (lane = row, 8 consecutive k per 16-deep
// step), loaded from HBM exactly once and normalised in place -- the normalised matrix never exists in memory.
// W streams through LDS in tiles of 64 k x 128 n (16 KB, three slots, one barrier per tile) copied with
// global_load_lds_dwordx4, and is read transposed (ds_read_b64_tr_b16) as the A operand:
//     C^T[n, r] += W^T[n, k] . LN(x)^T[k, r]
// so that a lane ends up with one output row and, per 32-column block, four runs of four consecutive columns -- the
// accumulator layout of the attention kernels.  A workgroup of 4 waves owns 128 rows and walks all of W once (two
// workgroups per CU): for each block of 128 output columns, d_model / 64 k tiles of 16 MFMAs per wave, then the
// epilogue (bias from LDS, SiLU for the u columns, rounding, a transposition through a per-wave LDS area so that
// every store instruction covers whole 128-byte lines).  W (2 MB for 512 x 2048) stays in every XCD's L2.
// Stores count in the same counter as the copies (vmcnt), so the wait after an epilogue leaves room for them.
#pragma once
#include "hstu_common.h"

namespace hstu {

struct UqvkFusedParams {
    const char* x;
    int64_t x_rs;  // elements
    const char* norm_weight;
    const char* norm_bias;
    float eps;
    const char* w;     // [K, n_out] row-major
    const char* bias;  // [n_out]
    char* out;         // [rows, n_out] dense
    int64_t rows;
    int n_out;   // multiple of 128
    int n_silu;  // multiple of 128: columns [0, n_silu) go through SiLU
    // Optional second output: the v | q | k columns (those from n_silu on) once more as e4m3 bytes,
    // out8[r, n - n_silu] = e4m3(rounded out[r, n] * inv_scale[t]), t = 0 (v: the next n_silu columns), 1 (q: the next
    // n_attn), 2 (k: the rest), clamped to +-448; and the largest |rounded out| of each of the three, for the scales of
    // the next batch.  NULL = off.
    unsigned char* out8;  // [rows, n_out - n_silu] dense
    float inv_scale[3];
    unsigned* absmax;     // [3]: bit patterns of non-negative floats, raised with atomicMax (the caller zeroes them)
    int n_attn;           // multiple of 64
};

constexpr int kUqvkWaves = 4, kUqvkRowsPerWave = 32;
constexpr int kUqvkTileK = 64, kUqvkTileN = 128;
constexpr int kUqvkSlot = kUqvkTileK * kUqvkTileN * 2;  // one W tile
constexpr int kUqvkBiasRing = 4 * 256;                  // the bias values of four consecutive column blocks
constexpr int kUqvkStageRow = 64 * 2 + 16;              // staging row: 64 outputs + pad
constexpr int kUqvkLds = 3 * kUqvkSlot + kUqvkBiasRing + kUqvkWaves * 32 * kUqvkStageRow;

// Chunk swizzle of a W tile (rows of 256 bytes = 16 chunks).  A transposing read touches rows {8g + 4sec + j}, j = 0..3,
// for the two half-waves g: the four rows of a half-wave go to four different 64-byte bank groups (row bits 0-1 ->
// chunk bits 2-3) and the two half-waves to different 32-byte halves of a group (row bit 3 -> chunk bit 1).
__device__ __forceinline__ int swz_w(int row) { return ((row & 3) << 2) | (((row >> 3) & 1) << 1); }

template <class TT, int KT>  // KT = d_model / 64: k tiles per column block
__global__ __launch_bounds__(kUqvkWaves * 64, 2) void hstu_uqvk_fused_kernel(const UqvkFusedParams p) {
    typedef typename TT::vec8 vec8;
    typedef typename TT::elem elem;
    constexpr int K = KT * kUqvkTileK, KS = K / 16;
    constexpr int NOPS = kUqvkTileK / 16 * 4;                  // A operands per tile: (kk, dt)
    constexpr int NPW = (kUqvkTileK * 16 / 64) / kUqvkWaves;  // copy instructions per wave and tile: 4
    constexpr int RG = kUqvkRowsPerWave / 32;                  // blocks of 32 rows per wave
    constexpr int PD = 3;
    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, l32 = lane & 31;
    const int64_t row0 = ((int64_t)blockIdx.x * kUqvkWaves + wave) * kUqvkRowsPerWave;  // first row of the wave
    const int nchunks = p.n_out / kUqvkTileN;
    const int ntiles = nchunks * KT;

    // copy of tile t = (column block c, k tile kt) into slot t % 3; wave 0 adds the block's bias values with the first k tile
    unsigned coff[NPW];
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
        const int pidx = (wave + kUqvkWaves * i) * 64 + lane;
        const int row = pidx >> 4;
        const int logical = (pidx & 15) ^ swz_w(row);
        coff[i] = (unsigned)row * (unsigned)(p.n_out * 2) + logical * 16;
    }
    auto issue_copy = [&](int t) {
        const int c = t / KT, kt = t - c * KT;
        char* slot = smem + (t % 3) * kUqvkSlot;
        const char* src = p.w + ((int64_t)kt * kUqvkTileK * p.n_out + (int64_t)c * kUqvkTileN) * 2;
#pragma unroll
        for (int i = 0; i < NPW; ++i) global_load_lds16_soff(src, coff[i], slot + (wave + kUqvkWaves * i) * 1024);
        // block c's bias is read after its last k tile, when at most the copies of block c + 1 have been issued
        if (kt == 0 && wave == 0 && lane < 16)
            global_load_lds16(p.bias + (int64_t)c * kUqvkTileN * 2 + lane * 16, smem + 3 * kUqvkSlot + (c & 3) * 256);
    };
    issue_copy(0);
    if (ntiles > 1) issue_copy(1);

    // ---- this wave's rows: load, normalise, keep as B operands
    vec8 xreg[RG][KS];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
        int64_t r = row0 + rg * 32 + l32;
        r = r < p.rows ? r : p.rows - 1;  // rows past the end repeat the last one; they are never stored
        const char* xp = p.x + (r * p.x_rs + 8 * g) * 2;
        float sum = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            xreg[rg][ks] = *(const vec8*)(xp + ks * 32);
#pragma unroll
            for (int j = 0; j < 8; ++j) sum += (float)xreg[rg][ks][j];
        }
        sum += __shfl_xor(sum, 32, 64);
        const float mean = sum * (1.0f / K);
        // the rows stay packed between the passes: without this the compiler keeps all their fp32 conversions alive
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xreg[rg][ks]));
        float sq = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float d = (float)xreg[rg][ks][j] - mean;
                sq += d * d;
            }
        sq += __shfl_xor(sq, 32, 64);
        const float rstd = __builtin_amdgcn_rsqf(sq * (1.0f / K) + p.eps);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xreg[rg][ks]));
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const vec8 wv = *(const vec8*)(p.norm_weight + (ks * 16 + 8 * g) * 2);
            const vec8 bv = *(const vec8*)(p.norm_bias + (ks * 16 + 8 * g) * 2);
            vec8 o;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (elem)(((float)xreg[rg][ks][j] - mean) * rstd * (float)wv[j] + (float)bv[j]);
            xreg[rg][ks] = o;
        }
    }

    // transposing reads of a W tile: lane supplies the address of 4 consecutive n of k row 8g + 4sec + j
    int waddr[2][4];
    {
        const int i16 = lane & 15, half = (lane >> 4) & 1, jrow = i16 >> 2, q4 = i16 & 3;
#pragma unroll
        for (int sec = 0; sec < 2; ++sec) {
            const int row = 8 * g + 4 * sec + jrow;  // + 16 kk
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                const int chunk = dt * 4 + 2 * half + (q4 >> 1);
                waddr[sec][dt] = row * 256 + ((chunk ^ swz_w(row)) * 16) + (q4 & 1) * 8;
            }
        }
    }
    char* stage = smem + 3 * kUqvkSlot + kUqvkBiasRing + wave * 32 * kUqvkStageRow;

    f32x16_t acc[RG][4];
    float amax[3] = {0.f, 0.f, 0.f};  // (e4m3 output) the largest |value| this lane has stored of v, q, k
    for (int c = 0; c < nchunks; ++c) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg)
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[rg][dt][r] = 0.f;
        const char* bias_lds = smem + 3 * kUqvkSlot + (c & 3) * 256;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            const int t = c * KT + kt;
            // everything but the newest batch of copies (tile t + 1) -- and, after an epilogue, its stores, which
            // count in the same counter -- has landed for this wave ...
            constexpr int STORES = RG * 8;
            if (t + 1 >= ntiles) __builtin_amdgcn_s_waitcnt(0x0F70);
            else if (kt == 0 && c > 0) __builtin_amdgcn_s_waitcnt(0x0F70 | ((NPW + STORES) & 15) | (((NPW + STORES) >> 4) << 14));
            else __builtin_amdgcn_s_waitcnt(0x0F70 | NPW);
            __syncthreads();  // ... and for every wave; nobody reads tile t - 1 any more, whose slot tile t + 2 takes
            if (t + 2 < ntiles) issue_copy(t + 2);
            const char* tile = smem + (t % 3) * kUqvkSlot;
            // NOPS A operands, each used for the wave's RG row blocks: op m = (kk, dt) = (m / 4, m % 4), requested PD ahead
            auto load_op = [&](int m) __attribute__((always_inline)) -> vec8 {
                const char* b = tile + (m >> 2) * 16 * 256;
                return read_vt_operand<TT>(b + waddr[0][m & 3], b + waddr[1][m & 3]);
            };
            vec8 fr[PD];
#pragma unroll
            for (int m = 0; m < PD; ++m) fr[m] = load_op(m);
#pragma unroll
            for (int m = 0; m < NOPS; ++m) {
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int rg = 0; rg < RG; ++rg) acc[rg][m & 3] = TT::mfma(fr[m % PD], xreg[rg][kt * (kUqvkTileK / 16) + (m >> 2)], acc[rg][m & 3]);
                if (m + PD < NOPS) fr[m % PD] = load_op(m + PD);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- epilogue of the column block: bias, SiLU for the u columns, rounding, transposition through LDS, stores
        const bool silu = c * kUqvkTileN < p.n_silu;
#pragma unroll
        for (int rg = 0; rg < RG; ++rg)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
            for (int d2 = 0; d2 < 2; ++d2) {
                const int dt = hf * 2 + d2;
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    typedef __attribute__((ext_vector_type(4))) elem elem4;
                    const elem4 b4 = *HSTU_LDS(const elem4, bias_lds + (dt * 32 + r4 * 8 + g * 4) * 2);
                    elem4 o4;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float v = acc[rg][dt][r4 * 4 + i] + (float)b4[i];
                        if (silu) v = v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
                        o4[i] = (elem)v;
                    }
                    *HSTU_LDS(elem4, stage + l32 * kUqvkStageRow + (d2 * 32 + r4 * 8 + g * 4) * 2) = o4;
                }
            }
            // 8 lanes cover one row's 128 bytes, 8 rows per instruction
            const int chunk = lane & 7, rsub = lane >> 3;
            const int col0 = c * kUqvkTileN + hf * 64;  // first column of this half block
            const bool to8 = p.out8 != nullptr && col0 >= p.n_silu;
            const int tensor = col0 < 2 * p.n_silu ? 0 : col0 < 2 * p.n_silu + p.n_attn ? 1 : 2;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = i * 8 + rsub;
                const i32x4_t v = *HSTU_LDS(const i32x4_t, stage + row * kUqvkStageRow + chunk * 16);
                if (row0 + rg * 32 + row < p.rows)
                    *(i32x4_t*)(p.out + ((row0 + rg * 32 + row) * p.n_out + col0) * 2 + chunk * 16) = v;
                if (to8) {
                    // the rounded values once more, scaled, as e4m3: 8 lanes cover 64 bytes of a row
                    const vec8 e = __builtin_bit_cast(vec8, v);
                    const float is = p.inv_scale[tensor];
                    float f[8], m8 = 0.f;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float x = (float)e[j];
                        m8 = __builtin_fmaxf(m8, __builtin_fabsf(x));
                        f[j] = __builtin_fminf(__builtin_fmaxf(x * is, -448.0f), 448.0f);
                    }
                    // (rows past the end repeat the last row: they change no maximum)
                    amax[0] = tensor == 0 ? __builtin_fmaxf(amax[0], m8) : amax[0];
                    amax[1] = tensor == 1 ? __builtin_fmaxf(amax[1], m8) : amax[1];
                    amax[2] = tensor == 2 ? __builtin_fmaxf(amax[2], m8) : amax[2];
                    int lo = 0, hi = 0;
                    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
                    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
                    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
                    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
                    if (row0 + rg * 32 + row < p.rows) {
                        typedef __attribute__((ext_vector_type(2))) int i32x2_t;
                        *(i32x2_t*)(p.out8 + (row0 + rg * 32 + row) * (int64_t)(p.n_out - p.n_silu) + (col0 - p.n_silu) + chunk * 8) = i32x2_t{lo, hi};
                    }
                }
            }
        }
    }
    if (p.out8 != nullptr) {
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            float m = amax[t];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) m = __builtin_fmaxf(m, __shfl_xor(m, d, 64));
            if (lane == 0 && m > 0.f) atomicMax(p.absmax + t, __builtin_bit_cast(unsigned, m));
        }
    }
}

}  // namespace hstu
