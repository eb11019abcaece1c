// Barrier-per-tile forward kernel: NW waves, each owning QT*32 query rows, all walking the same
// K/V tiles (double buffered in LDS), one workgroup per work item.  Generic in (dqk, dv) and the only kernel with an
// fp32 store: it serves unequal and 16-wide head dims and fp32 inputs; the pipelined kernels (hstu_fwd_pp_kernel.h,
// hstu_fwd_stream_kernel.h) take every other call.
// The scheme shared by both kernels is described at the top of hstu_common.h.
#pragma once
#include "hstu_common.h"

namespace hstu {

// One kv tile for one wave: S^T = K Q^T, P^T = s*sigmoid(alpha s) (masked if MASKED), O^T += V^T P^T.
// `sp0` is the sequence position of this lane's first kv slot: tile start + 4*(lane/32).
template <class TT, int DQK, int DV, int QT, int BN, int MASKED>
__device__ __forceinline__ void tile_compute(const char* kt, const char* vt, const typename TT::vec8 (&qreg)[QT][DQK / 16],
                                             f32x16_t (&oacc)[(DV + 31) / 32][QT], const int (&kaddr)[DQK / 16],
                                             const int (&vaddr)[2][(DV + 31) / 32], float c1, const SeqMask& M, int sp0,
                                             const RowMask (&rows)[QT]) {
    typedef typename TT::vec8 vec8;
    constexpr int NS = BN / 32, KS = DQK / 16, DT = (DV + 31) / 32, KROW = DQK * TT::ES, VROW = DV * TT::ES;
    // ---- S^T = K Q^T
    f32x16_t s[NS][QT];
#pragma unroll
    for (int sub = 0; sub < NS; ++sub) {
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[sub][qt][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            vec8 a = *HSTU_LDS(const vec8, kt + sub * 32 * KROW + kaddr[ks]);
#pragma unroll
            for (int qt = 0; qt < QT; ++qt) s[sub][qt] = TT::mfma(a, qreg[qt][ks], s[sub][qt]);
        }
    }
    // ---- P^T, packed to 16 bit
    vec8 pb[NS][QT][2];
#pragma unroll
    for (int sub = 0; sub < NS; ++sub)
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) silu_pack<TT, MASKED>(s[sub][qt], pb[sub][qt], c1, M, rows[qt], sp0 + sub * 32);
    // ---- O^T += V^T P^T
#pragma unroll
    for (int sub = 0; sub < NS; ++sub)
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const char* vb = vt + (sub * 32 + tt * 16) * VROW;
                vec8 a = read_vt_operand<TT>(vb + vaddr[0][dt], vb + vaddr[1][dt]);
#pragma unroll
                for (int qt = 0; qt < QT; ++qt) oacc[dt][qt] = TT::mfma(a, pb[sub][qt][tt], oacc[dt][qt]);
            }
}

template <class TT, int DQK, int DV, int QT, int NW, int BN, int OCC>
__global__ __launch_bounds__(NW * 64, OCC) void hstu_fwd_kernel(const FwdParams p) {
    typedef typename TT::vec8 vec8;
    constexpr int BM = NW * QT * 32;
    constexpr int KS = DQK / 16;
    constexpr int DT = (DV + 31) / 32;  // dv = 16 computes a 32-row tile and stores half of it
    constexpr int ES = TT::ES;
    constexpr int KROW = DQK * ES, VROW = DV * ES;
    constexpr int KTILE = BN * KROW, VTILE = BN * VROW, STAGE = KTILE + VTILE;
    constexpr int NT = NW * 64;
    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5;      // which half of the k-slots of an MFMA operand this lane holds
    const int l32 = lane & 31;    // operand row (A) / column (B, C) this lane holds

    Work W;
    if (!decode_work<BM, BN>(W, blockIdx.x)) return;
    const SeqMask& M = W.M;
    const int n = W.n;
    const int nq = W.m1;  // one past the last row of this item: rows from here on are never loaded or stored

    // rows of this wave, as sequence positions (inclusive; wR1 < wR0 if the wave has no rows)
    const int wq0 = W.m0 + wave * (QT * 32);
    const int wR0 = W.rbase + wq0;
    const int wR1 = (wq0 + QT * 32 < nq ? W.rbase + wq0 + QT * 32 : W.rbase + nq) - 1;

    int jt = next_valid_tile<BN>(W, W.jt_begin);
    const int jt_end = W.jt_end;

    const char* kbase = p.k + (W.seq_start * p.k_rs + (int64_t)W.h * p.k_hs) * ES;
    const char* vbase = p.v + (W.seq_start * p.v_rs + (int64_t)W.h * p.v_hs) * ES;
    const int64_t k_rsb = p.k_rs * ES, v_rsb = p.v_rs * ES;

    if (jt < jt_end) {
        load_tile_to_lds<BN, KROW, NT, false, ES>(kbase, k_rsb, jt * BN, n - 1, smem, wave, lane);
        load_tile_to_lds<BN, VROW, NT, true, ES>(vbase, v_rsb, jt * BN, n - 1, smem + KTILE, wave, lane);
    }

    vec8 qreg[QT][KS];
    const int64_t qrow0 = p.delta > 0 ? (int64_t)W.b * p.delta : W.seq_start;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) load_q_operand<TT, KS>(qreg[qt], p.q, qrow0, wq0 + qt * 32 + l32, nq, p.q_rs, p.q_hs, W.h, g, p.c1);

    RowMask rows[QT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) rows[qt].init(M, wR0 + qt * 32 + l32);

    int kaddr[KS];
    int vaddr[2][DT];
    lds_read_offsets<TT, DQK, DV>(kaddr, vaddr, lane);

    f32x16_t oacc[DT][QT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][qt][r] = 0.f;

    int stage = 0;
    while (jt < jt_end) {
        const int jn = next_valid_tile<BN>(W, jt + 1);

        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this tile's direct-to-LDS copies have landed
        __syncthreads();                      // ... for every wave, and the other stage is no longer read
        if (jn < jt_end) {
            char* nxt = smem + (stage ^ 1) * STAGE;
            load_tile_to_lds<BN, KROW, NT, false, ES>(kbase, k_rsb, jn * BN, n - 1, nxt, wave, lane);
            load_tile_to_lds<BN, VROW, NT, true, ES>(vbase, v_rsb, jn * BN, n - 1, nxt + KTILE, wave, lane);
        }

        const int cls = M.classify(wR0, wR1, jt * BN, BN);
        const char* kt = smem + stage * STAGE;
        if (cls == 2) {
            tile_compute<TT, DQK, DV, QT, BN, 0>(kt, kt + KTILE, qreg, oacc, kaddr, vaddr, p.c1, M, jt * BN + 4 * g, rows);
        } else if (cls == 1) {
            tile_compute<TT, DQK, DV, QT, BN, 1>(kt, kt + KTILE, qreg, oacc, kaddr, vaddr, p.c1, M, jt * BN + 4 * g, rows);
        }
        jt = jn;
        stage ^= 1;
    }

    const int64_t orow0 = p.delta > 0 ? (int64_t)W.b * p.delta : W.seq_start;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int ql = wq0 + qt * 32 + l32;
        store_output<TT, DT>(oacc, qt, p.o, orow0, ql, nq, p.o_rs, p.o_hs, W.h, g, output_scale(p, orow0 + (ql < nq ? ql : nq - 1)), DV);
    }
}

}  // namespace hstu
