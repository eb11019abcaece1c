// Key-stationary backward kernel (dK, dV) with the work on a block split between two waves of a SIMD.
//
// On this hardware a wave's VALU instructions hardly run in the shadow of its own MFMAs (measured: six VALU
// instructions behind every MFMA cost 10-20 of their 27 cycles, and the one-wave kernel's pointwise work came out
// fully on top of its products), while two waves of a SIMD do overlap.  The one-wave kernel cannot have a second
// wave per SIMD: K, V, dK and dV of 32 keys are 192 registers.  Here the eight waves of a workgroup form four pairs,
// waves w and w + 4 (they share SIMD w), and a pair shares 32 keys:
//     wave X (w):      S  = Q K^T         sigma, P (rounded, kept), G = slope (fp16, to LDS)       dV^T += dOut^T P
//     wave Y (w + 4):  dP = dOut V^T      dS = dP * G (rounded)                                    dK^T += Q^T dS
// so each holds one operand and one accumulator (96 registers), and each does two of the four products of a block.
// One barrier per block of 32 query rows keeps them a phase apart:
//     step s:   X: [S(s), dV(s-1)] then [pointwise(s) -> P(s), G(s)]     Y: [dS(s-1) from dP(s-1), G(s-1)] then [dK(s-1), dP(s)]
// X's long pointwise phase runs beside Y's products and Y's short one beside X's products.  G changes hands through
// two LDS buffers (written in step s, read in step s + 1).  Tiles of 64 query rows (Q and dOut) sit in three LDS
// slots; the Y waves, which have time to spare, copy them two tiles ahead.  A wave's LDS address registers carry the
// slot (moved on once per tile) and the block inside the tile is an instruction offset, so the reads cost no address
// arithmetic.  There is one loop body per kind of wave (the first tile is peeled): with one body per slot the
// register allocator moved the accumulators from region to region and spilled.
#pragma once
#include <type_traits>

#include "hstu_bwd_kernel.h"

namespace hstu {

constexpr int kBwdPpWaves = 8;

template <int DQK, int DV>
constexpr int bwd_pp_lds_bytes() {
    return 3 * kQueryTile * (DQK + DV) * 2 + 2 * 4 * 2048;
}

template <class TT, int DQK, int DV, bool STORE>
__global__ __launch_bounds__(kBwdPpWaves * 64, 1) void hstu_bwd_dkdv_pp_kernel(const BwdParams bp) {
    typedef typename TT::vec8 vec8;
    static_assert(DQK >= 32 && DV >= 32 && DQK % 32 == 0 && DV % 32 == 0, "a tile copy is at least one instruction per copying wave");
    const FwdParams& p = bp.f;
    constexpr int BN = kQueryTile, BM = kKeyBlock;
    constexpr int KS = DQK / 16, VS = DV / 16, DTK = DQK / 32, DTV = DV / 32;
    constexpr int QROW = DQK * 2, OROW = DV * 2;
    constexpr int QTILE = BN * QROW, OTILE = BN * OROW;
    constexpr int OREG = 3 * QTILE, GREG = 3 * (QTILE + OTILE), GBUF = 4 * 2048;  // LDS: Q slots, dOut slots, two G buffers
    constexpr int PD = 4;  // LDS operands in flight ahead of the MFMA that uses them
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int pr = wave & 3;  // the pair, and the pair's 32 keys
    const int g = lane >> 5, l32 = lane & 31;

    Work W;
    if (!bwd_decode<BM>(p, W, blockIdx.x, true)) return;
    const SeqMask& M = W.M;
    const int n = W.n;
    const int S0 = W.R0;           // first key row of the workgroup
    const int wS0 = S0 + pr * 32;  // first key row of the pair; it has no keys if wS0 >= n

    KeyBlockWalk walk;
    walk.init(M, p.targets != nullptr, S0, n);
    const int jt_end = walk.end;
    auto next_tile = [&](int jt) { return walk.next(M, jt, S0, n); };
    auto block_class = [&](int r0) { return block_class32(M, !walk.scan, r0, wS0, n); };

    KeyMask key;
    key.init(M, wS0 + l32);
    // Clear the entries of a packed block (first query row r0) that the mask removes: everything for class 0, the pairs
    // the predicate rejects for class 1.  Works on the rounded values, so whatever the pointwise step made of rows that
    // do not exist (even a NaN) goes away.
    auto apply_mask = [&](int cls, int r0, vec8 (&x)[2]) __attribute__((always_inline)) {
        if (cls == 2) return;
        const unsigned rows = cls == 1 ? key.valid_bits(r0 + 4 * g, n) : 0u;  // bit d: row r0 + 4 g + d sees the lane's key
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            u32x4_t m;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const int e = 8 * h + 2 * w, d = 8 * (e >> 2) + (e & 3);  // elements e, e + 1: rows d, d + 1
                const unsigned lo = (unsigned)__builtin_amdgcn_sbfe((int)rows, d, 1);
                const unsigned hi = (unsigned)__builtin_amdgcn_sbfe((int)rows, d + 1, 1);
                m[w] = (lo & 0xFFFFu) | (hi & 0xFFFF0000u);
            }
            x[h] = __builtin_bit_cast(vec8, __builtin_bit_cast(u32x4_t, x[h]) & m);
        }
    };
    // every LDS access of the step is complete for this wave, then for all of them
    auto step_barrier = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    int t_cur = next_tile(0);
    int t_nxt = t_cur < jt_end ? next_tile(t_cur + 1) : jt_end;
    int t_prev = t_cur;
    const bool any = t_cur < jt_end;

    // The visits of the walk: `tile(first, this tile, the one before, the one to copy, slot)` runs the two steps of a
    // tile, `drain()` the half step after the last one.  Both kinds of wave go through the same sequence, so they meet
    // at the same barriers.
    auto run = [&](auto&& tile, auto&& drain) __attribute__((always_inline)) {
        int t_nn = t_nxt < jt_end ? next_tile(t_nxt + 1) : jt_end;
        int slot = 0;
        tile(std::true_type{}, t_cur, t_prev, t_nn, slot);
        while (t_nxt < jt_end) {
            t_prev = t_cur;
            t_cur = t_nxt;
            t_nxt = t_nn;
            t_nn = t_nxt < jt_end ? next_tile(t_nxt + 1) : jt_end;
            slot = slot == 2 ? 0 : slot + 1;
            tile(std::false_type{}, t_cur, t_prev, t_nn, slot);
        }
        drain();
    };

    if (wave < 4) {
        // ================================================= X: S, P, G, dV =================================================
        vec8 kreg[KS];
        load_q_operand<TT, KS>(kreg, p.k, W.seq_start, wS0 + l32, n, p.k_rs, p.k_hs, W.h, g, p.c1);
        int qrow[KS], qtr[2][DTK], orow[VS], otr[2][DTV];
        lds_offsets_u<DQK>(qrow, qtr, lane);
        lds_offsets_u<DV>(orow, otr, lane);
        // qrow follows the slot of the tile whose S is formed; otr that of the block whose dV is formed: slot 2, the one
        // "before" the first, to start with
#pragma unroll
        for (int dt = 0; dt < DTV; ++dt) otr[0][dt] += OREG + 2 * OTILE, otr[1][dt] += OREG + 2 * OTILE;
        f32x16_t dvacc[DTV][1];
#pragma unroll
        for (int dt = 0; dt < DTV; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dvacc[dt][0][r] = 0.f;
        f32x16_t s;
        vec8 pb[2];
        char* gw = smem + GREG + pr * 2048 + lane * 16;

        // S of half H of the tile qrow points at (CUR) and dV of half HP of the tile otr points at (PREV), the two chains
        // alternating
        auto matrix = [&](auto h_, auto hp_, auto cur_, auto prev_) __attribute__((always_inline)) {
            constexpr int H = decltype(h_)::value, HP = decltype(hp_)::value;
            constexpr bool CUR = decltype(cur_)::value, PREV = decltype(prev_)::value;
            typedef TwoChains<CUR ? KS : 0, PREV ? 2 * DTV : 0> Ops;
            const char* qa = smem + H * 32 * QROW;
            const char* oa = smem + HP * 32 * OROW;
            auto load_op = [&](int k) __attribute__((always_inline)) -> vec8 {
                const int i = Ops::index(k);
                if (Ops::first(k)) return *HSTU_LDS(const vec8, qa + qrow[i]);
                const char* b = oa + (i / DTV) * 16 * OROW;
                return read_vt_operand<TT>(b + otr[0][i % DTV], b + otr[1][i % DTV]);
            };
            vec8 f[PD];
            if (CUR) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = 0.f;
            }
#pragma unroll
            for (int k = 0; k < PD && k < Ops::N; ++k) f[k] = load_op(k);
#pragma unroll
            for (int k = 0; k < Ops::N; ++k) {
                const int i = Ops::index(k);
                if (Ops::first(k)) s = TT::mfma(f[k % PD], kreg[i], s);
                else dvacc[i % DTV][0] = TT::mfma(f[k % PD], pb[i / DTV], dvacc[i % DTV][0]);
                if (k + PD < Ops::N) f[k % PD] = load_op(k + PD);
            }
        };
        // P (kept in pb, masked) and G (to LDS buffer `buf`) of the block whose first query row is r0
        auto pointwise = [&](int r0, int buf) __attribute__((always_inline)) {
            float pv[16], gv[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) silu_and_slope(s[e], pv[e], gv[e]);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float p8[8];
                u32x4_t g4;
#pragma unroll
                for (int j = 0; j < 8; ++j) p8[j] = pv[8 * h + j];
#pragma unroll
                for (int j = 0; j < 4; ++j) g4[j] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(gv[8 * h + 2 * j], gv[8 * h + 2 * j + 1]));
                pb[h] = TT::pack8(p8);
                *HSTU_LDS(u32x4_t, gw + buf * GBUF + h * 1024) = g4;
            }
            apply_mask(block_class(r0), r0, pb);
        };
        auto tile = [&](auto first_, int tj, int, int, int slot) __attribute__((always_inline)) {
            constexpr bool FIRST = decltype(first_)::value;
            // ---- block 0 of the tile; dV of block 1 of the tile before
            __builtin_amdgcn_s_setprio(3);
            matrix(I0{}, I1{}, std::true_type{}, std::integral_constant<bool, !FIRST>{});
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            pointwise(tj * BN, 0);
            {  // otr moves on to this tile
                const int d = slot == 0 ? -2 * OTILE : OTILE;
#pragma unroll
                for (int dt = 0; dt < DTV; ++dt) otr[0][dt] += d, otr[1][dt] += d;
            }
            __builtin_amdgcn_sched_barrier(0);
            step_barrier();
            // ---- block 1; dV of block 0
            __builtin_amdgcn_s_setprio(3);
            matrix(I1{}, I0{}, std::true_type{}, std::true_type{});
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            pointwise(tj * BN + 32, 1);
            {  // qrow moves on to the next tile
                const int d = slot == 2 ? -2 * QTILE : QTILE;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) qrow[ks] += d;
            }
            __builtin_amdgcn_sched_barrier(0);
            step_barrier();
        };
        auto drain = [&]() __attribute__((always_inline)) { matrix(I1{}, I1{}, std::false_type{}, std::true_type{}); };
        if (any) {
            step_barrier();
            run(tile, drain);
        }
        store_output<TT, DTV>(dvacc, 0, bp.dv, W.seq_start, wS0 + l32, n, bp.dv_rs, bp.dv_hs, W.h, g, bp.pscale, DV);
    } else {
        // ================================================= Y: dP, dS, dK =================================================
        const char* qbase = p.q + (W.seq_start * p.q_rs + (int64_t)W.h * p.q_hs) * 2;
        const char* obase = bp.dout + (W.seq_start * bp.do_rs + (int64_t)W.h * bp.do_hs) * 2;
        const int64_t q_rsb = p.q_rs * 2, o_rsb = bp.do_rs * 2;
        // Per-lane byte offsets of this wave's copies inside a tile (32 bits: the host chooses this kernel only when 64
        // rows stay far below 2 GB).  Instruction i of the wave covers rows (pr + 4 i) * RPI .. + RPI of the tile.
        constexpr int QCP = BN * (QROW / 16) / 64 / 4, OCP = BN * (OROW / 16) / 64 / 4, NCPW = QCP + OCP;
        constexpr int QRPI = 64 / (QROW / 16), ORPI = 64 / (OROW / 16);  // rows per instruction
        const int q_rsi = (int)q_rsb, o_rsi = (int)o_rsb;
        const int qlr = lane / (QROW / 16), olr = lane / (OROW / 16);    // the lane's row within an instruction
        unsigned qoff[QCP], ooff[OCP];
#pragma unroll
        for (int i = 0; i < QCP; ++i) {
            const int pos = (pr + i * 4) * 64 + lane, row = pos / (QROW / 16);
            qoff[i] = (unsigned)(row * q_rsi + (((pos % (QROW / 16)) ^ swz_u<QROW / 16>(row)) * 16));
        }
#pragma unroll
        for (int i = 0; i < OCP; ++i) {
            const int pos = (pr + i * 4) * 64 + lane, row = pos / (OROW / 16);
            ooff[i] = (unsigned)(row * o_rsi + (((pos % (OROW / 16)) ^ swz_u<OROW / 16>(row)) * 16));
        }
        // Every Y wave issues NCPW copy instructions per tile.  In a tile that reaches past the end of the sequence the
        // rows past the end re-read the last one (the mask removes them): their offset moves back by whole rows.
        auto copy_tile = [&](int jt, int slot) __attribute__((always_inline)) {
            char* ql = smem + slot * QTILE;
            char* ol = smem + OREG + slot * OTILE;
            const char* qb = qbase + (int64_t)jt * BN * q_rsb;
            const char* ob = obase + (int64_t)jt * BN * o_rsb;
            const int over = (jt + 1) * BN - n;  // rows of the tile past the end
            if (over <= 0) {
#pragma unroll
                for (int i = 0; i < QCP; ++i) global_load_lds16_soff(qb, qoff[i], ql + (pr + i * 4) * 1024);
#pragma unroll
                for (int i = 0; i < OCP; ++i) global_load_lds16_soff(ob, ooff[i], ol + (pr + i * 4) * 1024);
                return;
            }
            const int last = BN - 1 - over;  // last row of the tile inside the sequence
#pragma unroll
            for (int i = 0; i < QCP; ++i) {
                const int back = (pr + i * 4) * QRPI + qlr - last;
                global_load_lds16_soff(qb, qoff[i] - (unsigned)((back > 0 ? back : 0) * q_rsi), ql + (pr + i * 4) * 1024);
            }
#pragma unroll
            for (int i = 0; i < OCP; ++i) {
                const int back = (pr + i * 4) * ORPI + olr - last;
                global_load_lds16_soff(ob, ooff[i] - (unsigned)((back > 0 ? back : 0) * o_rsi), ol + (pr + i * 4) * 1024);
            }
        };
        if (any) copy_tile(t_cur, 0);
        if (t_nxt < jt_end) copy_tile(t_nxt, 1);
        vec8 vreg[VS];
        load_q_operand<TT, VS>(vreg, p.v, W.seq_start, wS0 + l32, n, p.v_rs, p.v_hs, W.h, g, 1.0f);
        int qrow[KS], qtr[2][DTK], orow[VS], otr[2][DTV];
        lds_offsets_u<DQK>(qrow, qtr, lane);
        lds_offsets_u<DV>(orow, otr, lane);
        // orow follows the slot of the tile whose dP is formed; qtr that of the block whose dK is formed (slot 2 at first)
#pragma unroll
        for (int vs = 0; vs < VS; ++vs) orow[vs] += OREG;
#pragma unroll
        for (int dt = 0; dt < DTK; ++dt) qtr[0][dt] += 2 * QTILE, qtr[1][dt] += 2 * QTILE;
        f32x16_t dkacc[DTK][1];
#pragma unroll
        for (int dt = 0; dt < DTK; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dkacc[dt][0][r] = 0.f;
        f32x16_t dp;
        vec8 dsb[2];
        const char* gr = smem + GREG + pr * 2048 + lane * 16;
        // stored-dS mode: this lane's slot in the blocks of the pair's 32 keys (block row 0 of the (sequence, head) pair)
        char* dsw = nullptr;
        if constexpr (STORE) dsw = ds_pair_base(bp, W, n) + (int64_t)(wS0 >> 5) * 2048 + (2 * l32 + g) * 16;
        const int64_t ds_qb_stride = (int64_t)bp.ds_pitch32 * 2048;

        // dK of half HP of the tile qtr points at (PREV) and dP of half H of the tile orow points at (CUR)
        auto matrix = [&](auto h_, auto hp_, auto cur_, auto prev_) __attribute__((always_inline)) {
            constexpr int H = decltype(h_)::value, HP = decltype(hp_)::value;
            constexpr bool CUR = decltype(cur_)::value, PREV = decltype(prev_)::value;
            typedef TwoChains<PREV ? 2 * DTK : 0, CUR ? VS : 0> Ops;
            const char* qa = smem + HP * 32 * QROW;
            const char* oa = smem + H * 32 * OROW;
            auto load_op = [&](int k) __attribute__((always_inline)) -> vec8 {
                const int i = Ops::index(k);
                if (!Ops::first(k)) return *HSTU_LDS(const vec8, oa + orow[i]);
                const char* b = qa + (i / DTK) * 16 * QROW;
                return read_vt_operand<TT>(b + qtr[0][i % DTK], b + qtr[1][i % DTK]);
            };
            vec8 f[PD];
            if (CUR) {
#pragma unroll
                for (int r = 0; r < 16; ++r) dp[r] = 0.f;
            }
#pragma unroll
            for (int k = 0; k < PD && k < Ops::N; ++k) f[k] = load_op(k);
#pragma unroll
            for (int k = 0; k < Ops::N; ++k) {
                const int i = Ops::index(k);
                if (Ops::first(k)) dkacc[i % DTK][0] = TT::mfma(f[k % PD], dsb[i / DTK], dkacc[i % DTK][0]);
                else dp = TT::mfma(f[k % PD], vreg[i], dp);
                if (k + PD < Ops::N) f[k % PD] = load_op(k + PD);
            }
        };
        // dS (rounded, masked, stored on request) of the block whose first query row is r0, from dP and the G in buffer `buf`
        auto pointwise = [&](int r0, int buf) __attribute__((always_inline)) -> int {
            const int cls = block_class(r0);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const u32x4_t g4 = *HSTU_LDS(const u32x4_t, gr + buf * GBUF + h * 1024);
                float d8[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const unsigned gj = g4[j];  // (a bit_cast of the vector element itself reads element 0)
                    const h2_t g2 = __builtin_bit_cast(h2_t, gj);
                    d8[2 * j] = dp[8 * h + 2 * j] * (float)g2[0];
                    d8[2 * j + 1] = dp[8 * h + 2 * j + 1] * (float)g2[1];
                }
                dsb[h] = TT::pack8(d8);
            }
            apply_mask(cls, r0, dsb);
            if constexpr (STORE) {
                if (cls != 0) {
                    char* dst = dsw + (r0 >> 5) * ds_qb_stride;
                    *(vec8*)dst = dsb[0];
                    *(vec8*)(dst + 1024 + (((2 * l32 + g) * 16) ^ 128) - (2 * l32 + g) * 16) = dsb[1];
                    return 2;
                }
            }
            return 0;
        };
        auto tile = [&](auto first_, int tj, int tp, int t_copy, int slot) __attribute__((always_inline)) {
            constexpr bool FIRST = decltype(first_)::value;
            // ---- dS and dK of block 1 of the tile before; dP of block 0 of this tile
            int stores = 0;  // store instructions of this tile's two steps
            if (!FIRST) stores += pointwise(tp * BN + 32, 1);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(3);
            matrix(I0{}, I1{}, std::true_type{}, std::integral_constant<bool, !FIRST>{});
            __builtin_amdgcn_s_setprio(0);
            {  // qtr moves on to this tile
                const int d = slot == 0 ? -2 * QTILE : QTILE;
#pragma unroll
                for (int dt = 0; dt < DTK; ++dt) qtr[0][dt] += d, qtr[1][dt] += d;
            }
            __builtin_amdgcn_sched_barrier(0);
            step_barrier();
            // ---- dS and dK of block 0; dP of block 1
            stores += pointwise(tj * BN, 0);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(3);
            matrix(I1{}, I0{}, std::true_type{}, std::true_type{});
            __builtin_amdgcn_s_setprio(0);
            {  // orow moves on to the next tile
                const int d = slot == 2 ? -2 * OTILE : OTILE;
#pragma unroll
                for (int vs = 0; vs < VS; ++vs) orow[vs] += d;
            }
            __builtin_amdgcn_sched_barrier(0);
            // The next tile, copied at the end of the tile before, has landed: everything but the stores of this tile
            // (memory instructions complete in order).  Then nobody reads the tile before this one any more (its last
            // readers finished before the barrier in the middle of this tile): the tile after next goes into its slot.
            if (stores == 4) __builtin_amdgcn_s_waitcnt(0x0F74);
            else if (stores == 2) __builtin_amdgcn_s_waitcnt(0x0F72);
            else __builtin_amdgcn_s_waitcnt(0x0F70);
            if (t_copy < jt_end) copy_tile(t_copy, slot == 0 ? 2 : slot - 1);
            step_barrier();
        };
        auto drain = [&]() __attribute__((always_inline)) {
            pointwise(t_cur * BN + 32, 1);
            __builtin_amdgcn_sched_barrier(0);
            matrix(I1{}, I1{}, std::false_type{}, std::true_type{});
        };
        if (any) {
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the first tiles have landed
            step_barrier();
            run(tile, drain);
        }
        store_output<TT, DTK>(dkacc, 0, bp.dk, W.seq_start, wS0 + l32, n, bp.dk_rs, bp.dk_hs, W.h, g, bp.gscale, DQK);
    }
}

}  // namespace hstu
