// Output projection of the attention block for gfx950 with the concatenation folded in:
//
//     out[r, :] = x[r, :] + [s0 | s1 | s2][r, :] @ W
//
// where the up to three column blocks of the left operand are separate matrices (u or SiLU(u), attn, and
// y = act(u) * norm(attn) as the norm-multiply kernel leaves it): `joined` of the reference (hstu_compute_output,
// ops/hstu_compute.py:107-214; ops/pytorch/pt_hstu_linear.py:87-124) is never written, two of its three blocks are
// read where they already are.
//
// A workgroup of 4 waves, one per SIMD, owns 256 rows and 256 of the output columns (a multiple of 256): wave (rh, cw) accumulates rows
// rh*128 .. +128 times columns cw*128 .. +128 of them, 4 x 4 MFMA blocks of 32 x 32 in 256 accumulator registers, so
// that an operand read from LDS feeds four MFMAs (half a KB of LDS reads per MFMA).  The workgroups of a row block
// run one after the other on the same XCD, so all but the first find the rows in that XCD's L2.
// The depth K = blocks * d is walked in tiles of 32.  Both operands come into LDS with global_load_lds_dwordx4 and
// nothing else touches them: W[32 k, 256 n] per tile (16 KB, two slabs of 128 columns in the format of the q/k/v
// producer, read transposed with ds_read_b64_tr_b16 as the A operand of  C^T[n, r] += W^T[n, k] . rows^T[k, r]) in
// a ring of four, issued two tiles before use; the rows in slices of two tiles (256 x 64, 32 KB: whole 128-byte
// lines, the eight chunks of a row swizzled with row / 2, read with ds_read_b128 as the B operand, lane = row) in a
// ring of three, issued two slices before use: with one wave per SIMD nothing but the depth of these rings
// hides the latency of L2 and HBM, and a tile lasts only half a microsecond.  One barrier per tile, between its two
// 16-deep steps, with the operands of the step behind it already in registers.  Every step is 16 MFMAs with exactly
// one memory instruction behind each (12 operand reads for the next step, 4 copy instructions): issued in bursts,
// the same instructions hold up the MFMA behind them and the kernel runs as the sum of its parts.  The epilogue turns
// the fp32 accumulators around in LDS (the rings are dead by then), adds the residual row-contiguously in fp32,
// rounds once and stores whole 128-byte lines.
#pragma once
#include <type_traits>

#include "hstu_common.h"
#include "hstu_uqvk_kernel.h"

namespace hstu {

struct OutputGemmParams {
    const char* src[3];  // the column blocks of the left operand, [rows, d] each
    int64_t src_rs[3];   // their row strides, elements
    int nsrc;            // 1 .. 3
    int d;               // columns per block: a multiple of 32
    const char* x;       // residual [rows, n]
    int64_t x_rs;
    const char* w;       // [nsrc * d, n] row-major
    char* out;           // [rows, n] dense
    int64_t rows;
    int n;               // output columns: a multiple of 256
    const char* bias;    // BIAS form: [n], added to every row; x is not read
    int n_silu;          // BIAS form: the first n_silu columns (a multiple of 256) go through SiLU
};

constexpr int kOutWaves = 4, kOutRows = 256, kOutWgCols = 256, kOutTileK = 32;
constexpr int kOutSliceK = 64;                          // the rows come in slices of two tiles: whole 128-byte lines
constexpr int kOutWSlot = kOutTileK * kOutWgCols * 2;  // 16 KB
constexpr int kOutASlot = kOutRows * kOutSliceK * 2;   // 32 KB
constexpr int kOutWRing = 4, kOutARing = 3;
constexpr int kOutLds = kOutWRing * kOutWSlot + kOutARing * kOutASlot;
constexpr int kOutStageRow = 64 * 4 + 16;  // staging row of the epilogue: 64 fp32 outputs + pad

// Workgroups b, b + 8, b + 16 ... land on the same XCD one after the other: they take the column blocks of one row
// block (row blocks in groups of eight, one per XCD).
__host__ __device__ inline long long output_gemm_grid(long long rows, int n) {
    const long long row_blocks = (rows + kOutRows - 1) / kOutRows;
    return (row_blocks + 7) / 8 * 8 * (n / kOutWgCols);
}

// Wait until at most N of the wave's copies into LDS are outstanding (they complete in order), then the barrier.
template <int N>
__device__ __forceinline__ void out_step_barrier() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}

// BIAS = false: out = x + rows @ W (the output projection).  BIAS = true: out = act(rows @ W + bias), act = SiLU on the
// first n_silu columns and nothing on the rest (the q/k/v producer's product for widths its own kernel does not take).
template <class TT, bool BIAS>
__global__ __launch_bounds__(kOutWaves * 64, 1) void hstu_output_gemm_kernel(const OutputGemmParams p) {
    typedef typename TT::vec8 vec8;
    typedef typename TT::elem elem;
    constexpr int NPW = (kOutWSlot / 1024) / kOutWaves;  // copy instructions per wave and 16 KB tile: 4
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    char* const a_ring = smem + kOutWRing * kOutWSlot;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5, l32 = lane & 31;
    const int rh = wave >> 1, cw = wave & 1;
    const unsigned ncb = (unsigned)p.n / kOutWgCols;  // column blocks of a row block
    const unsigned group = blockIdx.x / (8 * ncb), within = blockIdx.x - group * (8 * ncb);
    const int colblk = within >> 3;
    const int64_t row0 = ((int64_t)group * 8 + (within & 7)) * kOutRows;
    if (row0 >= p.rows) return;
    const int tpb = p.d / kOutTileK;  // tiles per block
    const int ntiles = p.nsrc * tpb;
    const int nslices = ntiles / 2;

    // ---- W copies: instruction i of this wave moves chunks (wave + 4 i) * 64 + lane of the tile (slab, k row, chunk)
    unsigned coff[NPW];
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
        const int pidx = (wave + kOutWaves * i) * 64 + lane;
        const int slab = pidx >> 9, row = (pidx >> 4) & 31;
        const int logical = (pidx & 15) ^ swz_w(row);
        coff[i] = (unsigned)row * (unsigned)(p.n * 2) + (colblk * 2 + slab) * 256 + logical * 16;
    }
    // (past the end: the last tile again, into a slot nobody reads -- the number of copies in flight is what the
    // waits count)
    int tw = 0;  // the W tile the next copy is for
    // (one instruction of the four at a time: they are issued between MFMAs)
    auto issue_w = [&](int i, int slot) __attribute__((always_inline)) {
        const int tc = tw < ntiles ? tw : ntiles - 1;
        const char* src = p.w + (int64_t)tc * kOutTileK * p.n * 2;
        global_load_lds16_soff(src, coff[i], smem + slot * kOutWSlot + (wave + kOutWaves * i) * 1024);
        if (i == NPW - 1) ++tw;
    };
    // ---- slice copies: a slice is 256 rows x 64 columns, 128-byte rows whose eight 16-byte chunks are swizzled with
    // the row; instruction i of this wave brings the 1 KB at byte (wave + 4 i) * 1024 of the slot, i.e. rows
    // (wave + 4 i) * 8 + lane / 8, physical chunk lane % 8, which holds the logical chunk lc
    const int lc = (lane & 7) ^ (((wave & 1) * 4 + (lane >> 4)) & 7);  // chunk ^ (row / 2) % 8
    // (the offsets of the block in progress: recomputed when the block changes, not picked from a table, which the
    // compiler would keep in scratch memory and wait for before every copy)
    int rrel[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int64_t r = row0 + (wave + kOutWaves * i) * 8 + (lane >> 3);
        r = r < p.rows ? r : p.rows - 1;  // rows past the end repeat the last one; they are never stored
        rrel[i] = (int)(r - row0);
    }
    int sb = 0, scol = 0, sn = 0;
    unsigned soff[8];
    const char* sbase;
    auto set_block = [&]() __attribute__((always_inline)) {
        const int64_t rs = sb == 0 ? p.src_rs[0] : (sb == 1 ? p.src_rs[1] : p.src_rs[2]);
        const char* s0 = sb == 0 ? p.src[0] : (sb == 1 ? p.src[1] : p.src[2]);
        sbase = s0 + row0 * rs * 2;
#pragma unroll
        for (int i = 0; i < 8; ++i) soff[i] = (unsigned)rrel[i] * (unsigned)(rs * 2) + lc * 16;
    };
    set_block();
    // (one instruction of the eight at a time)
    auto issue_slice = [&](int i, int slot) __attribute__((always_inline)) {
        global_load_lds16_soff(sbase + scol, soff[i], a_ring + slot * kOutASlot + (wave + kOutWaves * i) * 1024);
        if (i == 7 && ++sn < nslices) {  // (past the end: the last slice again)
            scol += kOutSliceK * 2;
            if (scol == p.d * 2) {
                scol = 0, sb = sb + 1 < p.nsrc ? sb + 1 : 0;
                set_block();
            }
        }
    };

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
                waddr[sec][dt] = cw * (32 * 256) + row * 256 + ((chunk ^ swz_w(row)) * 16) + (q4 & 1) * 8;
            }
        }
    }
    int baddr[2][2];  // B operands: row rh*128 + rb*32 + l32 of the slice, columns 32 half + 16 ks + 8 g .. +8
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int row = rh * 128 + l32;
            baddr[half][ks] = row * 128 + (((half * 4 + ks * 2 + g) ^ ((row >> 1) & 7)) * 16);
        }

    // accumulator element (dt, 4 r4 + i) of a lane is column dt*32 + r4*8 + g*4 + i of the wave's 128, for its row l32
    f32x16_t acc[4][4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            float init[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (BIAS) {  // the bias is where the sums start
                typedef __attribute__((ext_vector_type(4))) elem elem4;
                const elem4 b4 = *(const elem4*)(p.bias + (colblk * kOutWgCols + cw * 128 + dt * 32 + r4 * 8 + g * 4) * 2);
#pragma unroll
                for (int i = 0; i < 4; ++i) init[i] = (float)b4[i];
            }
#pragma unroll
            for (int rb = 0; rb < 4; ++rb)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[rb][dt][r4 * 4 + i] = init[i];
        }

    // The operands of the step in flight and of the one after.  A step is 16 MFMAs with one memory instruction behind
    // each: with one wave per SIMD an LDS read or a copy that is issued in a burst holds up the MFMA behind it, while
    // one at a time they disappear behind the 32 cycles of the MFMA before.  Slots 0 .. 3: the B operands of the next
    // step, 4 .. 11: the halves of its A operands, 12 .. 15: four copy instructions.
    s16x4_t flo[2][4], fhi[2][4];
    vec8 br[2][4];
    auto read_op = [&](int j, int wslot, int aslot, int half, int ks, s16x4_t(&lo)[4], s16x4_t(&hi)[4], vec8(&b)[4]) __attribute__((always_inline)) {
        const char* wt = smem + wslot * kOutWSlot + ks * 16 * 256;
        if (j < 4) b[j] = *HSTU_LDS(const vec8, a_ring + aslot * kOutASlot + baddr[half][ks] + j * 4096);
        else if (j & 1) hi[(j - 4) >> 1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(HSTU_LDS(s16x4_t, wt + waddr[1][(j - 4) >> 1]));
        else lo[(j - 4) >> 1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(HSTU_LDS(s16x4_t, wt + waddr[0][(j - 4) >> 1]));
    };
    auto mma = [&](int m, const s16x4_t(&lo)[4], const s16x4_t(&hi)[4], const vec8(&b)[4]) __attribute__((always_inline)) {
        const s16x8_t both = __builtin_shufflevector(lo[m >> 2], hi[m >> 2], 0, 1, 2, 3, 4, 5, 6, 7);
        acc[m & 3][m >> 2] = TT::mfma(__builtin_bit_cast(vec8, both), b[m & 3], acc[m & 3][m >> 2]);
    };

    // ---- prologue: W(0) and slice 0 first, then W(1), W(2), slice 1 and the first half of slice 2; only the first two
    // are waited for (every later wait leaves 16 copies outstanding, and at least 16 are issued behind each of these)
#pragma unroll
    for (int i = 0; i < NPW; ++i) issue_w(i, 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) issue_slice(i, 0);
#pragma unroll
    for (int t = 1; t < 3; ++t)
#pragma unroll
        for (int i = 0; i < NPW; ++i) issue_w(i, t);
#pragma unroll
    for (int i = 0; i < 8; ++i) issue_slice(i, 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) issue_slice(i, 2);
    out_step_barrier<2 * NPW + 8 + 4>();
#pragma unroll
    for (int j = 0; j < 12; ++j) read_op(j, 0, 0, 0, 0, flo[0], fhi[0], br[0]);

    // Tile t (half of slice t / 2).  Step A multiplies its first 16 columns, reads the operands of step B and issues the
    // copies of W(t + 3) into the slot of tile t - 1; the barrier publishes W(t + 1) and, for even t + 1, the next
    // slice (behind the copies of W(t + 1), issued in tile t - 2, came four copies in each of the four steps since:
    // the wait leaves those outstanding); step B multiplies the other 16 columns, reads the operands of tile t + 1
    // and issues half the copies of a slice: in the second tile of slice S the first half of slice S + 3 into the slot
    // of S, which every wave has finished reading, in the tile after it the second half.
    int wslot = 0, aslot = 0;  // t % 4, (t / 2) % 3
    auto tile = [&](auto Oddc) __attribute__((always_inline)) {
        constexpr bool ODD = decltype(Oddc)::value;
        const int wslot1 = (wslot + 1) & (kOutWRing - 1), wslot3 = (wslot + 3) & (kOutWRing - 1);
        const int aslot1 = ODD ? (aslot == kOutARing - 1 ? 0 : aslot + 1) : aslot;
        const int aslot_prev = aslot == 0 ? kOutARing - 1 : aslot - 1;
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            mma(m, flo[0], fhi[0], br[0]);
            __builtin_amdgcn_sched_barrier(0);
            if (m < 12) read_op(m, wslot, aslot, ODD, 1, flo[1], fhi[1], br[1]);
            else issue_w(m - 12, wslot3);
            __builtin_amdgcn_sched_barrier(0);
        }
        out_step_barrier<16>();
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            mma(m, flo[1], fhi[1], br[1]);
            __builtin_amdgcn_sched_barrier(0);
            if (m < 12) read_op(m, wslot1, aslot1, !ODD, 0, flo[0], fhi[0], br[0]);
            else if (ODD) issue_slice(m - 12, aslot);
            else issue_slice(m - 12 + 4, aslot_prev);
            __builtin_amdgcn_sched_barrier(0);
        }
        wslot = wslot1, aslot = aslot1;
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile(std::false_type{});
        tile(std::true_type{});
    }

    // ---- epilogue: fp32 accumulators through this wave's staging area (the rings are dead), + x, rounding, stores
    const int chunk = lane & 7, rsub = lane >> 3;  // 8 lanes cover one row's 64 columns, 8 rows per instruction
    const int col0 = colblk * kOutWgCols + cw * 128 + chunk * 8;
    vec8 xr[4][2][4];  // the residual of everything this lane stores, requested at once (rows past the end: the last row)
    if constexpr (!BIAS) {
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    int64_t r = row0 + rh * 128 + rb * 32 + i * 8 + rsub;
                    r = r < p.rows ? r : p.rows - 1;
                    xr[rb][hf][i] = *(const vec8*)(p.x + (r * p.x_rs + col0 + hf * 64) * 2);
                }
    }
    // the copies that are still on their way into the rings (repeats of the last tiles) have to land before the staging
    // areas take their place; the 32 loads of the residual behind them need not
    if constexpr (BIAS) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(32) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const bool silu = BIAS && colblk * kOutWgCols < p.n_silu;
    char* stage = smem + wave * 32 * kOutStageRow;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
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
                const int64_t r = row0 + rh * 128 + rb * 32 + row;
                const f32x4_t lo = *HSTU_LDS(const f32x4_t, stage + row * kOutStageRow + chunk * 32);
                const f32x4_t hi = *HSTU_LDS(const f32x4_t, stage + row * kOutStageRow + chunk * 32 + 16);
                if (r < p.rows) {
                    vec8 ov;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if constexpr (BIAS) {
                            const float a0 = lo[j], a1 = hi[j];
                            ov[j] = (elem)(silu ? a0 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * a0)) : a0);
                            ov[4 + j] = (elem)(silu ? a1 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * a1)) : a1);
                        } else {
                            ov[j] = (elem)(lo[j] + (float)xr[rb][hf][i][j]);
                            ov[4 + j] = (elem)(hi[j] + (float)xr[rb][hf][i][4 + j]);
                        }
                    }
                    *(vec8*)(p.out + (r * p.n + col0 + hf * 64) * 2) = ov;
                }
            }
        }
}

}  // namespace hstu
