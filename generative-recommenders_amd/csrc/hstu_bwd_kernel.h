// Backward of the HSTU jagged attention for gfx950: dq, dk, dv from dout (full attention only).
//
// With x = alpha * s, s = q . k, sigma = sigmoid(x) and M the mask:
//     P  = M * x * sigma / N                      out = P V
//     dV = P^T dOut
//     dP = dOut V^T
//     dS = M * dP * sigma * (1 + x * (1 - sigma)) / N
//     dQ = alpha * dS K        dK = alpha * dS^T Q
// (what _hstu_attn_bwd_one_block of the reference computes, ops/triton/triton_hstu_attention.py:1905-2021; like it,
// P and dS are rounded to the operand type before their products, and the constant factors are applied to the fp32
// sums at the end).  Nothing is saved by the forward pass: the scores are recomputed.
//
// Two kernels, each with the structure of the barrier-per-tile forward kernel (hstu_fwd_kernel.h) and without
// atomics, so the result does not depend on the schedule:
//   * hstu_bwd_dkdv_kernel: a workgroup owns 128 key rows (K and V of 32 rows per wave in registers, K pre-scaled
//     by c1 = -alpha * log2(e)) and walks the query rows that can see them in tiles of 64 (Q and dOut through LDS):
//         S[q, kv]   = Q K^T          A = Q tile (row reads),            B = K registers
//         dP[q, kv]  = dOut V^T       A = dOut tile (row reads),         B = V registers
//         dV^T[dv, kv] += dOut^T P    A = dOut tile (transposing reads), B = P packed from the accumulator
//         dK^T[d, kv]  += Q^T dS      A = Q tile (transposing reads),    B = dS packed
//   * hstu_bwd_dq_kernel: a workgroup owns 128 query rows (Q pre-scaled and dOut in registers) and walks the key
//     rows as the forward kernel does:
//         S^T[kv, q]  = K Q^T         A = K tile (row reads),            B = Q registers
//         dP^T[kv, q] = V dOut^T      A = V tile (row reads),            B = dOut registers
//         dQ^T[d, q] += K^T dS^T      A = K tile (transposing reads),    B = dS^T packed
// A tile that is read both by rows (ds_read_b128) and transposed (ds_read_b64_tr_b16) is stored with one chunk
// swizzle that keeps both kinds of read off each other's banks (swz_u below).
#pragma once
#include <type_traits>

#include "hstu_common.h"

namespace hstu {

struct BwdParams {
    FwdParams f;  // q, k, v with strides, offsets, targets, mask integers, c1, num_mb, pairs_per_xcd, order; `o` unused
    const char* dout;
    char *dq, *dk, *dv;
    int64_t do_rs, do_hs, dq_rs, dq_hs, dk_rs, dk_hs, dv_rs, dv_hs;  // strides in elements
    float pscale;  // dV = pscale * sum(p dOut), p = t * sigma with t = c1 * s:  (alpha / N) / c1
    float gscale;  // dQ, dK = gscale * sum(...):  alpha / N
};

// Chunk swizzle for a tile read both ways: the bits the transposing read needs (swz_v) plus row bit 3 in chunk bit 0,
// which makes the 16 rows of a ds_read_b128 land in 16 different 16-byte slots and changes nothing for a transposing
// read (all rows one such instruction touches agree in bit 3).
template <int CH>
__device__ __forceinline__ int swz_u(int row) {
    static_assert(CH == 2 || CH == 4 || CH == 8 || CH == 16, "row of 32 .. 256 bytes");
    if (CH == 2) return 0;
    return swz_v<CH, 2>(row) | ((row >> 3) & 1);
}

template <int ROWS, int ROWBYTES, int NTHREADS>
__device__ __forceinline__ void load_tile_u(const char* gbase, int64_t row_stride_bytes, int row0, int last_row, char* lds_tile,
                                            int wave, int lane) {
    constexpr int CH = ROWBYTES / 16;
    constexpr int INSTR = ROWS * CH / 64;
    constexpr int NWAVES = NTHREADS / 64;
#pragma unroll
    for (int i = 0; i < (INSTR + NWAVES - 1) / NWAVES; ++i) {
        const int inst = wave + i * NWAVES;
        if (inst >= INSTR) break;
        const int p = inst * 64 + lane;
        const int row = p / CH;
        const int logical = (p % CH) ^ swz_u<CH>(row);
        int grow = row0 + row;
        grow = grow > last_row ? last_row : grow;  // rows past the end re-read the last one; the mask removes them
        global_load_lds16(gbase + (int64_t)grow * row_stride_bytes + logical * 16, lds_tile + inst * 1024);
    }
}

// Byte offsets of this lane's reads inside a block of 32 tile rows of D 16-bit elements: `rowaddr[ks]` for the A
// operand "row lane%32, elements 16 ks + 8 (lane/32) .. +8", `traddr[sec][dt]` for the transposed A operand (32
// columns dt*32.. x 16 rows) as in lds_read_offsets of the forward kernels.
template <int D>
__device__ __forceinline__ void lds_offsets_u(int (&rowaddr)[D / 16], int (&traddr)[2][(D + 31) / 32], int lane) {
    constexpr int ROW = D * 2, CH = ROW / 16, DT = (D + 31) / 32;
    const int g = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) rowaddr[ks] = l32 * ROW + (((2 * ks + g) ^ swz_u<CH>(l32)) * 16);
    const int i16 = lane & 15, half = (lane >> 4) & 1, jrow = i16 >> 2, q4 = i16 & 3;
#pragma unroll
    for (int sec = 0; sec < 2; ++sec) {
        const int row = 8 * sec + 4 * g + jrow;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int chunk = dt * 4 + 2 * half + (q4 >> 1);
            traddr[sec][dt] = row * ROW + ((chunk ^ swz_u<CH>(row)) * 16) + (q4 & 1) * 8;
        }
    }
}

// The sequence of (b, h) and the block of BM rows an item stands for; `low_first`: block 0 first (the heaviest
// for the key-stationary kernel: every later row sees it), else the last block first.
template <int BM>
__device__ __forceinline__ bool bwd_decode(const FwdParams& p, Work& w, int bid, bool low_first) {
    const int xcd = bid & 7, slot = bid >> 3;
    const int pair_local = slot / p.num_mb;
    const int j = slot - pair_local * p.num_mb;
    const int mb = low_first ? j : p.num_mb - 1 - j;
    const int pair = pair_local * 8 + xcd;
    if (pair >= p.B * p.H) return false;
    const int rseq = pair / p.H;
    w.h = pair - rseq * p.H;
    w.b = p.order ? HSTU_CONST(int, p.order)[rseq] : rseq;
    int64_t seq_start, seq_end;
    if (p.offsets_i64) {
        seq_start = HSTU_CONST(int64_t, p.offsets)[w.b];
        seq_end = HSTU_CONST(int64_t, p.offsets)[w.b + 1];
    } else {
        seq_start = HSTU_CONST(int, p.offsets)[w.b];
        seq_end = HSTU_CONST(int, p.offsets)[w.b + 1];
    }
    w.seq_start = uniform64(seq_start);
    int n = __builtin_amdgcn_readfirstlane((int)(seq_end - seq_start));
    n = n > p.max_seq_len ? p.max_seq_len : n;
    w.n = w.nq = n;
    w.m0 = mb * BM;
    w.rbase = 0;
    if (n <= 0 || w.m0 >= n) return false;
    int t = 0;
    if (p.targets) t = p.targets_i64 ? (int)HSTU_CONST(int64_t, p.targets)[w.b] : HSTU_CONST(int, p.targets)[w.b];
    t = __builtin_amdgcn_readfirstlane(t);
    SeqMask& M = w.M;
    M.n = n;
    M.w = p.w;
    M.c = p.c;
    M.f = p.f;
    M.shift = p.c > 0 ? p.c - 1 : 0;
    w.u = n - t;
    M.max_id = w.u - M.shift;
    M.idclamp = p.targets ? M.max_id : 0x7fffffff;
    w.R0 = w.m0;
    w.R1 = (w.m0 + BM < n ? w.m0 + BM : n) - 1;
    w.split = 0;
    w.nsplit = 1;
    w.block_id = 0;
    w.skip_scan = p.w > 0 || p.c > 0 || p.targets != nullptr;
    return true;
}

// sigma and its companions for one score: t = c1 * s = -x * log2(e).
//   p = t * sigma                      (P up to the constant 1 / (c1 * N) * alpha)
//   g = sigma * (1 + x * (1 - sigma))  = sigma + ln2 * p * (sigma - 1)
__device__ __forceinline__ void silu_and_slope(float t, float& p, float& g) {
    const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
    p = t * sig;
    g = __builtin_fmaf(0.6931471805599453f * p, sig - 1.0f, sig);
}

// ---- key-stationary kernel: dK, dV ---------------------------------------------------------------------------------

// Per-lane constants of the mask predicate for one key.
struct KeyMask {
    int pos, ids;
    __device__ __forceinline__ void init(const SeqMask& M, int key_pos) {
        pos = key_pos;
        ids = M.id(key_pos);
    }
    // rows at or past the end of the sequence are padding of the last tile
    __device__ __forceinline__ bool valid(const SeqMask& M, int row_pos) const {
        const int idr = M.id(row_pos);
        const int wr = (M.w == 0 || (M.f > 0 && idr >= M.max_id - M.f)) ? 0x7fffffff : M.w;
        const bool ok = (row_pos == pos) | ((unsigned)(idr - ids - 1) < (unsigned)wr) | ((M.c > 0) & (idr == 0) & (ids < M.max_id));
        return ok & (row_pos < M.n);
    }
};

// Order in which two chains of NA and NB accumulating MFMAs are issued: alternately while both last, so that
// neighbours never depend on each other.
template <int NA, int NB>
struct TwoChains {
    static constexpr int N = NA + NB;
    static constexpr int M = NA < NB ? NA : NB;
    static constexpr bool first(int k) { return k < 2 * M ? (k & 1) == 0 : NA > NB; }
    static constexpr int index(int k) { return k < 2 * M ? k / 2 : k - M; }
};

// The key-stationary kernel has two 128-row accumulators and K, V in registers: one wave per SIMD.  A wave alone
// must therefore overlap its own matrix and VALU work, which it does by software pipelining over blocks of 32
// query rows: phase A issues the S and dP products of the NEXT block, one MFMA at a time, each followed by the
// pointwise work (sigmoid, slope, mask, rounding) on one accumulator element of the CURRENT block; phase B then
// issues the dV and dK products of the current block.  LDS operands are requested PD MFMAs ahead.  Tiles of 64
// query rows sit in three LDS slots; the one barrier per tile comes after the first block of a tile has gone through
// phase B, when nobody can still read the tile before it, whose slot the next copy overwrites.
// Blocks are skipped per wave only in whole phases (a block with no valid pair for the wave's keys gets neither
// products nor pointwise work); the barrier count per tile is the same for every wave.
template <class TT, int DQK, int DV, int NW, int BN>
__global__ __launch_bounds__(NW * 64, 1) void hstu_bwd_dkdv_kernel(const BwdParams bp) {
    typedef typename TT::vec8 vec8;
    static_assert(BN == 64, "two blocks of 32 query rows per tile");
    const FwdParams& p = bp.f;
    constexpr int BM = NW * 32;  // key rows per workgroup
    constexpr int KS = DQK / 16, VS = DV / 16, DTK = (DQK + 31) / 32, DTV = (DV + 31) / 32;
    constexpr int QROW = DQK * 2, OROW = DV * 2;
    constexpr int QTILE = BN * QROW, OTILE = BN * OROW, STAGE = QTILE + OTILE;
    constexpr int NT = NW * 64;
    constexpr int PD = 3;  // LDS operands in flight ahead of the MFMA that uses them
    typedef TwoChains<KS, VS> OpsA;
    typedef TwoChains<2 * DTV, 2 * DTK> OpsB;
    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, l32 = lane & 31;

    Work W;
    if (!bwd_decode<BM>(p, W, blockIdx.x, true)) return;
    const SeqMask& M = W.M;
    const int n = W.n;
    const int S0 = W.R0, S1 = W.R1;  // key rows of the workgroup (inclusive)
    const int wS0 = S0 + wave * 32;  // first key row of the wave; the wave has no keys if wS0 > S1

    // query tiles [.., jt_end): rows at or after the first key (all rows if a contextual prefix sees every key), up
    // to the last row whose window still reaches the block (targets sit at id max_id)
    int q_hi = n - 1;
    if (M.w > 0 && M.f == 0) {
        const int id1 = M.id(S1);
        const bool targets_reach = p.targets != nullptr && M.max_id - id1 <= M.w;
        if (!targets_reach) {
            const int hi = id1 + M.w + M.shift;
            q_hi = hi < q_hi ? hi : q_hi;
        }
    }
    const int jt_end = q_hi / BN + 1;
    auto next_tile = [&](int jt) {
        if (W.skip_scan)
            while (jt < jt_end) {
                const int r1 = (jt + 1) * BN < n ? (jt + 1) * BN - 1 : n - 1;
                if (M.classify(jt * BN, r1, S0, BM) != 0) break;
                ++jt;
            }
        return jt;
    };

    const char* qbase = p.q + (W.seq_start * p.q_rs + (int64_t)W.h * p.q_hs) * 2;
    const char* obase = bp.dout + (W.seq_start * bp.do_rs + (int64_t)W.h * bp.do_hs) * 2;
    const int64_t q_rsb = p.q_rs * 2, o_rsb = bp.do_rs * 2;
    auto copy_tile = [&](int jt, int slot) {
        load_tile_u<BN, QROW, NT>(qbase, q_rsb, jt * BN, n - 1, smem + slot * STAGE, wave, lane);
        load_tile_u<BN, OROW, NT>(obase, o_rsb, jt * BN, n - 1, smem + slot * STAGE + QTILE, wave, lane);
    };

    int t_cur = next_tile(M.c > 0 ? 0 : S0 / BN);
    int t_nxt = t_cur < jt_end ? next_tile(t_cur + 1) : jt_end;
    if (t_cur < jt_end) copy_tile(t_cur, 0);
    if (t_nxt < jt_end) copy_tile(t_nxt, 1);

    vec8 kreg[KS], vreg[VS];
    load_q_operand<TT, KS>(kreg, p.k, W.seq_start, wS0 + l32, n, p.k_rs, p.k_hs, W.h, g, p.c1);
    load_q_operand<TT, VS>(vreg, p.v, W.seq_start, wS0 + l32, n, p.v_rs, p.v_hs, W.h, g, 1.0f);
    KeyMask key;
    key.init(M, wS0 + l32);

    int qrow[KS], qtr[2][DTK], orow[VS], otr[2][DTV];
    lds_offsets_u<DQK>(qrow, qtr, lane);
    lds_offsets_u<DV>(orow, otr, lane);

    f32x16_t dkacc[DTK][1], dvacc[DTV][1];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
#pragma unroll
        for (int dt = 0; dt < DTK; ++dt) dkacc[dt][0][r] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DTV; ++dt) dvacc[dt][0][r] = 0.f;
    }

    // class of the block of 32 query rows starting at r0 against this wave's keys: 0 nothing valid, 1 masked, 2 all valid
    auto block_class = [&](int r0) {
        if (r0 >= n || wS0 > S1) return 0;
        const int r1 = r0 + 31 < n ? r0 + 31 : n - 1;
        int cls = M.classify(r0, r1, wS0, 32);
        if (cls == 2 && r0 + 31 >= n) cls = 1;
        return cls;
    };

    // Phase A.  MFMA: issue S and dP of the block whose Q / dOut rows start at qn / on into (s_n, dp_n).
    // PW (0 none, 1 masked, 2 all valid): P and dS of the block held in (s_c, dp_c), whose first query row is r0_c,
    // packed into pb / dsb.
    auto phase_a = [&](auto mfma_c, auto pw_c, const char* qn, const char* on, f32x16_t& s_n, f32x16_t& dp_n, const f32x16_t& s_c,
                       const f32x16_t& dp_c, int r0_c, vec8 (&pb)[2], vec8 (&dsb)[2]) __attribute__((always_inline)) {
        constexpr bool MFMA = decltype(mfma_c)::value;
        constexpr int PW = decltype(pw_c)::value;
        constexpr int NA = OpsA::N;
        auto load_op = [&](int k) __attribute__((always_inline)) -> vec8 {
            return OpsA::first(k) ? *HSTU_LDS(const vec8, qn + qrow[OpsA::index(k)]) : *HSTU_LDS(const vec8, on + orow[OpsA::index(k)]);
        };
        vec8 fr[PD];
        if constexpr (MFMA) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s_n[r] = dp_n[r] = 0.f;
#pragma unroll
            for (int k = 0; k < PD && k < NA; ++k) fr[k] = load_op(k);
        }
        float pv[16], dsv[16];
#pragma unroll
        for (int k = 0; k < NA; ++k) {
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MFMA) {
                if (OpsA::first(k)) s_n = TT::mfma(fr[k % PD], kreg[OpsA::index(k)], s_n);
                else dp_n = TT::mfma(fr[k % PD], vreg[OpsA::index(k)], dp_n);
                if (k + PD < NA) fr[k % PD] = load_op(k + PD);
            }
            if constexpr (PW != 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    if (e * NA / 16 != k) continue;
                    float pr, gr;
                    silu_and_slope(s_c[e], pr, gr);
                    float dsr = dp_c[e] * gr;
                    if constexpr (PW == 1) {
                        const bool ok = key.valid(M, r0_c + 8 * (e >> 2) + 4 * g + (e & 3));
                        pr = ok ? pr : 0.f;
                        dsr = ok ? dsr : 0.f;
                    }
                    pv[e] = pr;
                    dsv[e] = dsr;
                    if (e == 7 || e == 15) {
                        float p8[8], d8[8];
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            p8[j] = pv[e - 7 + j];
                            d8[j] = dsv[e - 7 + j];
                        }
                        pb[e >> 3] = TT::pack8(p8);
                        dsb[e >> 3] = TT::pack8(d8);
                    }
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // Phase B: dV^T += dOut^T P and dK^T += Q^T dS for the block whose rows start at qc / oc.
    auto phase_b = [&](const char* qc, const char* oc, const vec8 (&pb)[2], const vec8 (&dsb)[2]) __attribute__((always_inline)) {
        constexpr int NB = OpsB::N;
        auto load_op = [&](int k) __attribute__((always_inline)) -> vec8 {
            const int i = OpsB::index(k);
            if (OpsB::first(k)) {
                const char* b = oc + (i / DTV) * 16 * OROW;
                return read_vt_operand<TT>(b + otr[0][i % DTV], b + otr[1][i % DTV]);
            }
            const char* b = qc + (i / DTK) * 16 * QROW;
            return read_vt_operand<TT>(b + qtr[0][i % DTK], b + qtr[1][i % DTK]);
        };
        vec8 fr[PD];
#pragma unroll
        for (int k = 0; k < PD && k < NB; ++k) fr[k] = load_op(k);
#pragma unroll
        for (int k = 0; k < NB; ++k) {
            __builtin_amdgcn_sched_barrier(0);
            const int i = OpsB::index(k);
            if (OpsB::first(k)) dvacc[i % DTV][0] = TT::mfma(fr[k % PD], pb[i / DTV], dvacc[i % DTV][0]);
            else dkacc[i % DTK][0] = TT::mfma(fr[k % PD], dsb[i / DTK], dkacc[i % DTK][0]);
            if (k + PD < NB) fr[k % PD] = load_op(k + PD);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    typedef std::integral_constant<bool, true> Yes;
    typedef std::integral_constant<bool, false> No;
    typedef std::integral_constant<int, 0> Pw0;
    typedef std::integral_constant<int, 1> Pw1;
    typedef std::integral_constant<int, 2> Pw2;
    // phase A with the two choices made at run time (both are wave-uniform)
    auto run_a = [&](bool mfma, int pw, const char* qn, const char* on, f32x16_t& s_n, f32x16_t& dp_n, const f32x16_t& s_c,
                     const f32x16_t& dp_c, int r0_c, vec8 (&pb)[2], vec8 (&dsb)[2]) __attribute__((always_inline)) {
        if (mfma) {
            if (pw == 2) phase_a(Yes{}, Pw2{}, qn, on, s_n, dp_n, s_c, dp_c, r0_c, pb, dsb);
            else if (pw == 1) phase_a(Yes{}, Pw1{}, qn, on, s_n, dp_n, s_c, dp_c, r0_c, pb, dsb);
            else phase_a(Yes{}, Pw0{}, qn, on, s_n, dp_n, s_c, dp_c, r0_c, pb, dsb);
        } else {
            if (pw == 2) phase_a(No{}, Pw2{}, qn, on, s_n, dp_n, s_c, dp_c, r0_c, pb, dsb);
            else if (pw == 1) phase_a(No{}, Pw1{}, qn, on, s_n, dp_n, s_c, dp_c, r0_c, pb, dsb);
        }
    };

    if (t_cur < jt_end) {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the first tiles have landed
        __syncthreads();
        f32x16_t sx, dpx, sy, dpy;  // block 0 of a tile lives in x, block 1 in y
        vec8 pb[2], dsb[2];
        int slot = 0;
        int clsx = block_class(t_cur * BN);
        run_a(clsx != 0, 0, smem, smem + QTILE, sx, dpx, sx, dpx, 0, pb, dsb);
        while (true) {
            const char* qt = smem + slot * STAGE;
            const char* ot = qt + QTILE;
            // block 1 of this tile enters phase A while block 0 gets its pointwise work
            const int clsy = block_class(t_cur * BN + 32);
            run_a(clsy != 0, clsx, qt + 32 * QROW, ot + 32 * OROW, sy, dpy, sx, dpx, t_cur * BN, pb, dsb);
            if (clsx != 0) phase_b(qt, ot, pb, dsb);
            const bool more = t_nxt < jt_end;
            int t_nn = jt_end;
            if (more) {
                __builtin_amdgcn_s_waitcnt(0x0F70);  // the next tile, copied during the last one, has landed
                __syncthreads();                      // ... for every wave; and nobody reads the tile before this one any more
                t_nn = next_tile(t_nxt + 1);
                const int nslot = slot == 2 ? 0 : slot + 1;
                if (t_nn < jt_end) copy_tile(t_nn, nslot == 2 ? 0 : nslot + 1);
                clsx = block_class(t_nxt * BN);
                const char* qn = smem + nslot * STAGE;
                run_a(clsx != 0, clsy, qn, qn + QTILE, sx, dpx, sy, dpy, t_cur * BN + 32, pb, dsb);
            } else {
                run_a(false, clsy, qt, ot, sx, dpx, sy, dpy, t_cur * BN + 32, pb, dsb);
            }
            if (clsy != 0) phase_b(qt + 32 * QROW, ot + 32 * OROW, pb, dsb);
            if (!more) break;
            t_cur = t_nxt;
            t_nxt = t_nn;
            slot = slot == 2 ? 0 : slot + 1;
        }
    }
    store_output<TT, DTK>(dkacc, 0, bp.dk, W.seq_start, wS0 + l32, n, bp.dk_rs, bp.dk_hs, W.h, g, bp.gscale, DQK);
    store_output<TT, DTV>(dvacc, 0, bp.dv, W.seq_start, wS0 + l32, n, bp.dv_rs, bp.dv_hs, W.h, g, bp.pscale, DV);
}

// ---- query-stationary kernel: dQ -----------------------------------------------------------------------------------

template <class TT, int DQK, int DV, int NW, int BN>
__global__ __launch_bounds__(NW * 64, 2) void hstu_bwd_dq_kernel(const BwdParams bp) {
    typedef typename TT::vec8 vec8;
    const FwdParams& p = bp.f;
    constexpr int BM = NW * 32;
    constexpr int KS = DQK / 16, VS = DV / 16, DTK = (DQK + 31) / 32;
    constexpr int KROW = DQK * 2, VROW = DV * 2;
    constexpr int KTILE = BN * KROW, VTILE = BN * VROW, STAGE = KTILE + VTILE;
    constexpr int NT = NW * 64;
    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, l32 = lane & 31;

    Work W;
    if (!bwd_decode<BM>(p, W, blockIdx.x, false)) return;
    const SeqMask& M = W.M;
    const int n = W.n;
    kv_tile_range(M, W.u, W.R0, W.R1, BN, W.jt_begin, W.jt_end);

    const int wq0 = W.m0 + wave * 32;
    const int wR0 = wq0;
    const int wR1 = (wq0 + 32 < n ? wq0 + 32 : n) - 1;

    int jt = next_valid_tile<BN>(W, W.jt_begin);
    const int jt_end = W.jt_end;

    const char* kbase = p.k + (W.seq_start * p.k_rs + (int64_t)W.h * p.k_hs) * 2;
    const char* vbase = p.v + (W.seq_start * p.v_rs + (int64_t)W.h * p.v_hs) * 2;
    const int64_t k_rsb = p.k_rs * 2, v_rsb = p.v_rs * 2;

    if (jt < jt_end) {
        load_tile_u<BN, KROW, NT>(kbase, k_rsb, jt * BN, n - 1, smem, wave, lane);
        load_tile_u<BN, VROW, NT>(vbase, v_rsb, jt * BN, n - 1, smem + KTILE, wave, lane);
    }

    vec8 qreg[KS], doreg[VS];
    load_q_operand<TT, KS>(qreg, p.q, W.seq_start, wq0 + l32, n, p.q_rs, p.q_hs, W.h, g, p.c1);
    load_q_operand<TT, VS>(doreg, bp.dout, W.seq_start, wq0 + l32, n, bp.do_rs, bp.do_hs, W.h, g, 1.0f);
    RowMask row;
    row.init(M, wR0 + l32);

    int krow[KS], ktr[2][DTK], vrow[VS], vtr_unused[2][(DV + 31) / 32];
    lds_offsets_u<DQK>(krow, ktr, lane);
    lds_offsets_u<DV>(vrow, vtr_unused, lane);

    f32x16_t dqacc[DTK][1];
#pragma unroll
    for (int dt = 0; dt < DTK; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dqacc[dt][0][r] = 0.f;

    int stage = 0;
    while (jt < jt_end) {
        const int jn = next_valid_tile<BN>(W, jt + 1);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (jn < jt_end) {
            char* nxt = smem + (stage ^ 1) * STAGE;
            load_tile_u<BN, KROW, NT>(kbase, k_rsb, jn * BN, n - 1, nxt, wave, lane);
            load_tile_u<BN, VROW, NT>(vbase, v_rsb, jn * BN, n - 1, nxt + KTILE, wave, lane);
        }
        const char* kt = smem + stage * STAGE;
        const char* vt = kt + KTILE;
#pragma unroll
        for (int sub = 0; sub < BN / 32; ++sub) {
            const int s0 = jt * BN + sub * 32;  // first key row of the block of 32
            const int cls = M.classify(wR0, wR1, s0, 32);
            if (cls == 0) continue;
            f32x16_t s, dp;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s = TT::mfma(*HSTU_LDS(const vec8, kt + sub * 32 * KROW + krow[ks]), qreg[ks], s);
#pragma unroll
            for (int ks = 0; ks < VS; ++ks) dp = TT::mfma(*HSTU_LDS(const vec8, vt + sub * 32 * VROW + vrow[ks]), doreg[ks], dp);
            vec8 dsb[2];
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                float d8[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int r = half * 8 + j;
                    float pr, gr;
                    silu_and_slope(s[r], pr, gr);
                    float dsr = dp[r] * gr;
                    if (cls == 1) dsr = row.valid(M, s0 + 8 * (r >> 2) + 4 * g + (r & 3)) ? dsr : 0.f;
                    d8[j] = dsr;
                }
                dsb[half] = TT::pack8(d8);
            }
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const char* kb = kt + (sub * 32 + tt * 16) * KROW;
#pragma unroll
                for (int dt = 0; dt < DTK; ++dt)
                    dqacc[dt][0] = TT::mfma(read_vt_operand<TT>(kb + ktr[0][dt], kb + ktr[1][dt]), dsb[tt], dqacc[dt][0]);
            }
        }
        jt = jn;
        stage ^= 1;
    }
    store_output<TT, DTK>(dqacc, 0, bp.dq, W.seq_start, wq0 + l32, n, bp.dq_rs, bp.dq_hs, W.h, g, bp.gscale, DQK);
}

}  // namespace hstu
