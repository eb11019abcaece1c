// One-group pipelined forward kernel (tile config 3) and the building blocks it shares with the streaming two-group
// kernel of hstu_fwd_stream_kernel.h (tile copies through buffer descriptors, the Q rows by LDS-DMA).
//
// Per score element the matrix cores need 512 flops (half a cycle per element and SIMD at peak) while
// s*sigmoid(alpha s) needs about 30 VALU issue cycles per 64 elements -- the two cost the same, and a wave
// that has just issued an MFMA cannot issue VALU work for a while, so the two kinds of work must come from
// different waves of a SIMD at the same time.  Here they come from the two workgroups that share a CU (4 waves
// and 128 query rows each): a workgroup runs, per kv tile, a matrix phase (O^T += V^T P^T of the previous tile
// interleaved with S^T = K Q^T of this one) and then the VALU phase of the same tile (P^T from S^T), one barrier
// per tile, and nothing aligns the two workgroups, so that one's matrix phases fall on the other's VALU phases
// most of the time.  The streaming kernel holds two wave groups of ONE workgroup half a step apart on purpose.
//
// The matrix phase is one straight line of MFMAs whose LDS operands are requested PD MFMAs ahead
// (rotating registers, order pinned with sched_barrier) so that one wave alone keeps its matrix core fed.
// Tiles are never skipped per wave: a tile with nothing valid for a wave's rows just gets P^T = 0.
//
// LDS holds two K tiles and two V tiles.  The first tiles and the Q rows come with the prologue; from step 1 on,
// step i copies V(i) and K(i+1) from inside its matrix phase (spread between MFMAs) and waits for them at its own
// end.  The scheme common to all kernels is described at the top of hstu_common.h.
#pragma once
#include <type_traits>

#include "hstu_common.h"

namespace hstu {

// Direct HBM -> LDS copy of one tile, spread over four waves (in the two-group kernel the four "A" waves: copies issued
// from the "B" waves' matrix phase were measured to stall it; from the A waves they are free), through a buffer descriptor of the sequence's K (or V)
// rows for this head: rows past the end of the sequence arrive as zeros.  A lane keeps ONE byte offset per kind of tile:
// the instructions of a wave lie 256 / CH rows apart, which is a multiple of every swizzle's period, so instruction i
// differs from instruction 0 only by a number of whole rows, and that goes into the wave-uniform offset together with
// the tile's first row -- a copy is issued between MFMAs, where every further instruction counts, and costs three
// scalar instructions besides the copy itself.
template <int ROWS, int ROWBYTES, bool IS_V, int ES>
struct TileCopy {
    static constexpr int CH = ROWBYTES / 16;
    static constexpr int NI = ROWS * CH / 64;       // wave-wide copy instructions per tile
    static constexpr int NCW = 4;                   // waves that issue copies
    static constexpr int PER_WAVE = (NI + NCW - 1) / NCW;
    static constexpr int STEP = NCW * 64 / CH;      // rows between two instructions of one wave
    unsigned off0;  // this lane's offset from the tile's first row in the wave's first instruction
    __device__ __forceinline__ void init(int wave, int lane, unsigned row_stride_bytes) {
        const int row = (wave * 64 + lane) / CH;
        const int phys = lane % CH;  // (64 is a multiple of CH)
        const int logical = phys ^ (IS_V ? swz_v<CH, ES>(row) : swz_k<CH>(row));
        off0 = (unsigned)row * row_stride_bytes + logical * 16;
    }
    // Copy instruction `i` (0 .. PER_WAVE-1) of this wave for the tile starting at row `row0` of the sequence that
    // `rsrc` describes.
    __device__ __forceinline__ void issue_one(int i, i32x4_t rsrc, unsigned row_stride_bytes, int row0, char* lds_tile, int wave) const {
        const int inst = wave + NCW * i;
        if (inst < NI) buffer_load_lds16(rsrc, off0, (unsigned)(row0 + i * STEP) * row_stride_bytes, lds_tile + inst * 1024);
    }
    __device__ __forceinline__ void issue(i32x4_t rsrc, unsigned row_stride_bytes, int row0, char* lds_tile, int wave) const {
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) issue_one(i, rsrc, row_stride_bytes, row0, lds_tile, wave);
    }
};

// Copy of 32 rows of Q (the wave's own, from row `q0` of the rows `rsrc` describes) into `stage`, laid out like 32 rows
// of a K tile (16-byte chunks XOR-ed with the row number), so that the operand is read back with the K tile's offsets.
// Rows past the end of the sequence arrive as zeros.
template <int ROWBYTES>
__device__ __forceinline__ void copy_q_rows(i32x4_t rsrc, unsigned row_stride_bytes, int q0, char* stage, int lane) {
    constexpr int CH = ROWBYTES / 16;   // chunks per row
    constexpr int RPI = 64 / CH;        // rows per copy instruction
    const int r = lane / CH, phys = lane % CH;
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
        const unsigned o = (unsigned)r * row_stride_bytes + (phys ^ swz_k<CH>(i * RPI + r)) * 16;
        buffer_load_lds16(rsrc, o, (unsigned)(q0 + i * RPI) * row_stride_bytes, stage + i * 1024);
    }
}

// The multiplication by -alpha*log2(e) that load_q_operand applies to 16-bit rows.
template <class TT, int KS>
__device__ __forceinline__ void prescale_q(typename TT::vec8 (&qreg)[KS], float qscale) {
    if constexpr (TT::PRESCALE_Q) {
        typedef typename TT::elem elem;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) qreg[ks][j] = (elem)((float)qreg[ks][j] * qscale);
    }
}

// NG = 1 (the only instantiation): a single wave group, 4 waves, 128 rows, 2 LDS slots, two workgroups per CU and one
// barrier per tile.  It wastes less than 256-row blocks on short sequences, whose last block would be mostly empty.
template <class TT, int DQK, int DV, int BN, int NG>
__global__ __launch_bounds__(NG * 256, 2) void hstu_fwd_pp_kernel(const FwdParams p_arg) {
    typedef typename TT::vec8 vec8;
    static_assert(DQK == DV, "the interleaved matrix phase assumes as many first-product as second-product MFMAs");
    static_assert(NG == 1, "the two-group form is hstu_fwd_stream_kernel");
    constexpr int BM = 128;
    constexpr int NS = BN / 32;
    constexpr int KS = DQK / 16;
    constexpr int DT = DV / 32;
    constexpr int ES = TT::ES;
    constexpr int KROW = DQK * ES, VROW = DV * ES;
    constexpr int KTILE = BN * KROW, VTILE = BN * VROW;
    constexpr int NSLOT = 2;
    // LDS: NSLOT K slots, then NSLOT V slots.  A static array (the only LDS object, so it sits at address 0) lets
    // every tile and slot offset fold into the immediate field of the LDS reads.
    // 16 more bytes at the end carry the next work item's number from thread 0 to the rest of the workgroup.
    __shared__ __attribute__((aligned(1024))) char smem[NSLOT * (KTILE + VTILE) + 16];
    constexpr int NEXT_OFF = NSLOT * (KTILE + VTILE);
    constexpr int VOFF = NSLOT * KTILE;
    // The immediate offset of an LDS read reaches 64 KB.  K reads stay below that; V reads go through address
    // registers biased by VBIAS so that VOFF - VBIAS + slot and tile offsets fit the immediate as well.
    constexpr int VBIAS = (NSLOT * (KTILE + VTILE) > 65536) ? 32768 : 0;
    static_assert(VOFF >= VBIAS && VOFF - VBIAS + NSLOT * VTILE <= 65536 && NSLOT * KTILE <= 65536, "LDS immediates");
    // 8-bit operands: four 16-deep operands make one 64-deep MFMA at twice the rate (needs dqk % 64 == 0 and a
    // 64-row kv tile)
    constexpr bool WIDE = ES == 1 && DQK % 64 == 0 && BN == 64;
    constexpr int NOPS = WIDE ? (NS * KS + NS * 2 * DT) / 4 : NS * KS + NS * 2 * DT;   // MFMAs of one matrix phase
    constexpr int PD = NOPS >= 16 ? 6 : 4;        // operands in flight (16-deep scheme)

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5;
    const int l32 = lane & 31;

    // Persistent workgroups: the grid holds as many workgroups as the chip keeps resident, and each takes work
    // items (heaviest first) until none is left.  This spares the launch of a workgroup per item (2-3 us of an
    // idle CU slot each time).  Item ids are slot * 8 + xcd: the items of one XCD's list share K/V through that
    // XCD's L2.  With a queue (one counter per XCD in the caller's workspace, set to the number of workgroups per
    // XCD before the launch) the next item is whatever the counter of the workgroup's own XCD hands out, asked for
    // at the start of the current item so that the answer is there at its end; when that list is exhausted the
    // workgroup goes on with the lists of the other XCDs (the XCDs do not run equally fast, and a ragged batch
    // does not split evenly).  Without a queue the items of the own list are dealt with a stride, in alternating
    // direction from round to round, so that a workgroup that got the heaviest item of one round gets the
    // lightest of the next.
    const int GL = gridDim.x >> 3, lw = blockIdx.x >> 3, xcd = blockIdx.x & 7;
    // with work lists the number of items of an XCD is what the plan kernel counted
    const int slots_per_xcd = p_arg.nitems ? HSTU_CONST(int, p_arg.nitems)[xcd] : p_arg.slots_per_xcd;
    int* const queue = p_arg.queue;
    int round = 0;
    int bid = lw < slots_per_xcd ? lw * 8 + xcd : -1;
    auto process_item = [&]() __attribute__((always_inline)) {
    // Per-lane values that depend on the lane number only are recomputed for every item (a few dozen VALU
    // instructions): hoisted out of the item loop they would be spilled.  The empty asm hides from the compiler
    // that the lane number is the same every time.
    int lane_v = lane;
    asm volatile("" : "+v"(lane_v));
    // The parameters are read from the kernel argument segment again for every item (scalar loads that hit the
    // scalar cache): held in registers across the loop, they and everything the compiler derives from them
    // ahead of the loop would not fit the scalar register file.
    const __attribute__((address_space(4))) FwdParams* pk =
        (const __attribute__((address_space(4))) FwdParams*)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(pk));
    const FwdParams& p = *(const FwdParams*)pk;
    Work W;
    if (!decode_work<BM, BN>(W, bid)) return;
    const SeqMask& M = W.M;
    const int n = W.n;
    const int nq = W.m1;  // one past the last row of this item: rows from here on are never loaded or stored

    const int wq0 = W.m0 + wave * 32;
    const int wR0 = W.rbase + wq0;
    const int wR1 = (wq0 + 32 < nq ? W.rbase + wq0 + 32 : W.rbase + nq) - 1;

    // Tiles [full_begin, full_end) are valid in every element for this wave's rows (no mask code): the tile
    // lies strictly before the first row's id and inside every row's window.  Every other tile takes the
    // exact per-element predicate, and so does a sequence that breaks the caller contract
    // "non-target positions >= contextual_seq_len" (ids would go negative).
    int full_begin = 0, full_end = 0;
    if (wR1 >= wR0 && W.u >= p.c && W.u >= 0) {
        const int idr_lo = M.id(wR0), idr_hi = M.id(wR1);
        full_end = (idr_lo + M.shift) / BN;          // keys s with s - shift < id(first row)
        if (full_end * BN > n) full_end = n / BN;
        if (p.w > 0 && idr_hi - p.w > 0) full_begin = (idr_hi - p.w + M.shift + BN - 1) / BN;
    }

    // This kernel walks the contiguous tile range [jt_begin, jt_end): a tile inside it that holds no valid
    // pair (other targets' columns of a target row block) is computed and masked to zero rather than
    // skipped, which keeps the step count known up front and the loop free of side exits.
    // no window, contextual prefix or targets: the mask of a diagonal tile is just "key <= row" (rows of the
    // last, partly filled row block that lie past the sequence end are never stored, so they need no mask)
    const bool plain_causal = p.w == 0 && p.c == 0 && p.targets == nullptr;
    const int jt_end = W.jt_end;
    const int T = jt_end - W.jt_begin;  // steps
    const int64_t orow0 = p.delta > 0 ? (int64_t)W.b * p.delta : W.seq_start;
    float* const my_partial = p.kv_splits > 1 ? p.partial + (int64_t)W.split * p.partial_stride : nullptr;
    if (T <= 0) return;  // cannot happen for a row block with rows (each row sees itself); kept for safety
    int t_cur = W.jt_begin;

    // descriptors of the sequence's K and V rows for this head (the host keeps rows * stride below 2^32)
    const unsigned k_rsb = (unsigned)p.k_rs * ES, v_rsb = (unsigned)p.v_rs * ES;
    const i32x4_t kbase = make_buffer_rsrc(p.k + (W.seq_start * p.k_rs + (int64_t)W.h * p.k_hs) * ES, (unsigned)n * k_rsb);
    const i32x4_t vbase = make_buffer_rsrc(p.v + (W.seq_start * p.v_rs + (int64_t)W.h * p.v_hs) * ES, (unsigned)n * v_rsb);
    typedef TileCopy<BN, KROW, false, ES> KCopy;
    typedef TileCopy<BN, VROW, true, ES> VCopy;
    KCopy kcopy;
    VCopy vcopy;
    kcopy.init(wave, lane_v, k_rsb);
    vcopy.init(wave, lane_v, v_rsb);
    constexpr int NPW = KCopy::PER_WAVE + VCopy::PER_WAVE;  // copy instructions per wave and step
    static_assert(NPW <= 15 && NOPS % NPW == 0, "vmcnt immediate / even spread of the copies");

    // Copy schedule.  Before step 0: K(t0) -> K slot 0, V(t0) -> V slot 0, K(t1) -> K slot 1.  Step i >= 1 copies V(i)
    // and K(i+1) and waits for them at its own end (step 0 copies nothing: its tiles came with the prologue, so that
    // the first steps of a workgroup do not each expose a memory latency).
    // One group: the wave's 32 Q rows come by LDS-DMA as well, into the second slot pair, which is empty until the
    // first step (two waves' rows fill a K slot, two a V slot), laid out like rows of a K tile so that they are read back
    // with the K tile's offsets.  Fetched with per-lane loads (32 rows x 32 bytes per instruction) the same rows hold
    // the CU's vector-memory path some 400 cycles per wave; the copy of the second K tile moves behind the barrier that
    // follows, where it still has all of the first step to land.
    constexpr bool Q_BY_DMA = DQK == DV;
    constexpr int QW = 32 * KROW;  // bytes of a wave's Q rows
    const int64_t qrow0 = p.delta > 0 ? (int64_t)W.b * p.delta : W.seq_start;
    char* const qstage = smem + (wave < 2 ? KTILE + wave * QW : VOFF + VTILE + (wave - 2) * QW);
    if constexpr (Q_BY_DMA) {
        static_assert(2 * QW == KTILE && KTILE == VTILE, "two waves' rows per slot");
        const unsigned q_rsb = (unsigned)p.q_rs * ES;
        copy_q_rows<KROW>(make_buffer_rsrc(p.q + (qrow0 * p.q_rs + (int64_t)W.h * p.q_hs) * ES, (unsigned)W.nq * q_rsb), q_rsb, wq0, qstage,
                          lane_v);
    }
    kcopy.issue(kbase, k_rsb, t_cur * BN, smem, wave);
    vcopy.issue(vbase, v_rsb, t_cur * BN, smem + VOFF, wave);
    if constexpr (!Q_BY_DMA) kcopy.issue(kbase, k_rsb, (t_cur + 1 < jt_end ? t_cur + 1 : t_cur) * BN, smem + KTILE, wave);

    vec8 qreg[KS];
    if constexpr (!Q_BY_DMA) load_q_operand<TT, KS>(qreg, p.q, qrow0, wq0 + l32, nq, p.q_rs, p.q_hs, W.h, g, p.c1);
    RowMask row;
    row.init(M, wR0 + l32);

    int kaddr[KS];
    int vaddr[2][DT];
    lds_read_offsets<TT, DQK, DV>(kaddr, vaddr, lane_v);
    // (only vaddr[0] is kept: the second transposing read of an operand lies 8 rows below the first for every lane,
    // which is an immediate)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        vaddr[0][dt] += VBIAS;
        asm volatile("" : "+v"(vaddr[0][dt]));  // keep the bias in the register, out of the immediates
    }

    f32x16_t oacc[DT][1];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][0][r] = 0.f;

    f32x16_t s[NS];        // S^T of the tile in flight between this wave's matrix and VALU phases
    vec8 pb[NS][2];        // P^T of the tile in flight between its VALU phase and its next matrix phase

    if constexpr (Q_BY_DMA) {
        // the Q rows were asked for first: they have landed when only the first tiles' copies are outstanding
        // (a tile of fewer copy instructions than copying waves leaves some waves without one: those wait for everything)
        constexpr int LEAVE = (KCopy::NI % KCopy::NCW == 0 && VCopy::NI % VCopy::NCW == 0) ? KCopy::PER_WAVE + VCopy::PER_WAVE : 0;
        __builtin_amdgcn_s_waitcnt((LEAVE & 0xF) | ((LEAVE >> 4) << 14) | 0x0F70);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qreg[ks] = *HSTU_LDS(const vec8, qstage + kaddr[ks]);
        prescale_q<TT, KS>(qreg, p.c1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // ... and are in registers before the barrier lets the slots go
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    if constexpr (Q_BY_DMA) kcopy.issue(kbase, k_rsb, (t_cur + 1 < jt_end ? t_cur + 1 : t_cur) * BN, smem + KTILE, wave);

    // ---- building blocks ------------------------------------------------------------------------------
    // Copy instruction j (0 .. NPW-1) of the step of list entry i (SLOT = i % 2): the V tile of entry i, then the K
    // tile of entry i+1.  Past the end of the list the last entry is copied again (redundant, but it keeps the
    // number of copy instructions per step constant).
    auto issue_copy = [&](auto slot_c, int j) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        const int tv = t_cur < jt_end ? t_cur : jt_end - 1;
        const int tk = t_cur + 1 < jt_end ? t_cur + 1 : jt_end - 1;
        if (j < VCopy::PER_WAVE)
            vcopy.issue_one(j, vbase, v_rsb, tv * BN, smem + VOFF + SLOT * VTILE, wave);
        else
            kcopy.issue_one(j - VCopy::PER_WAVE, kbase, k_rsb, tk * BN, smem + ((SLOT + 1) % NSLOT) * KTILE, wave);
    };
    // S^T = K Q^T only (first step), K slot chosen at run time.
    auto gemm1_only = [&](int kslot) __attribute__((always_inline)) {
        const char* kt = smem + kslot * KTILE;
#pragma unroll
        for (int sub = 0; sub < NS; ++sub) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[sub][r] = 0.f;
            if constexpr (WIDE) {
#pragma unroll
                for (int k4 = 0; k4 < KS / 4; ++k4) {
                    vec8 a[4], b[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        a[j] = *HSTU_LDS(const vec8, kt + sub * 32 * KROW + kaddr[4 * k4 + j]);
                        b[j] = qreg[4 * k4 + j];
                    }
                    s[sub] = TT::mfma64(a, b, s[sub]);
                }
            } else {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    vec8 a = *HSTU_LDS(const vec8, kt + sub * 32 * KROW + kaddr[ks]);
                    s[sub] = TT::mfma(a, qreg[ks], s[sub]);
                }
            }
        }
    };
    // O^T += V^T P^T only (after the last step), V slot chosen at run time.
    auto gemm2_only = [&](int vslot) __attribute__((always_inline)) {
        const char* vt = smem + (VOFF - VBIAS) + vslot * VTILE;
        if constexpr (WIDE) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                vec8 a[4], b[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {  // j = 2 sub + tt: the whole 64-row tile in one MFMA
                    const char* vb = vt + ((j >> 1) * 32 + (j & 1) * 16) * VROW;
                    a[j] = read_vt_operand<TT>(vb + vaddr[0][dt], vb + vaddr[0][dt] + 8 * VROW);
                    b[j] = pb[j >> 1][j & 1];
                }
                oacc[dt][0] = TT::mfma64(a, b, oacc[dt][0]);
            }
        } else {
#pragma unroll
            for (int sub = 0; sub < NS; ++sub)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const char* vb = vt + (sub * 32 + tt * 16) * VROW;
                        vec8 a = read_vt_operand<TT>(vb + vaddr[0][dt], vb + vaddr[0][dt] + 8 * VROW);
                        oacc[dt][0] = TT::mfma(a, pb[sub][tt], oacc[dt][0]);
                    }
        }
    };
    // Full matrix phase of list entry i (SLOT = i % 3): second product of entry i-1 interleaved with the
    // first product of entry i, plus this wave's share of the step's copies.
    // MFMA k: even k -> second product (sub, tt, dt) = ((k/2)/(2 DT), ((k/2)/DT) % 2, (k/2) % DT);
    //         odd k  -> first product  (ks, sub) = ((k/2)/NS, (k/2) % NS).
    auto matrix_phase = [&](auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        const char* kt = smem + SLOT * KTILE;
        const char* vt = smem + (VOFF - VBIAS) + ((SLOT + NSLOT - 1) % NSLOT) * VTILE;
        if constexpr (WIDE) {
            // MFMA m: even m -> second product, dv tile m/2, all four (sub, tt) quarters of the kv tile at once;
            //         odd m  -> first product, (k slab of 64, sub) = ((m/2)/NS, (m/2) % NS).
            // The operands of MFMA m+1 are requested before MFMA m is issued.
            auto load_group = [&](int m, vec8 (&a)[4]) __attribute__((always_inline)) {
                const int o = m >> 1;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if ((m & 1) == 0) {
                        const char* vb = vt + ((j >> 1) * 32 + (j & 1) * 16) * VROW;
                        a[j] = read_vt_operand<TT>(vb + vaddr[0][o], vb + vaddr[0][o] + 8 * VROW);
                    } else {
                        a[j] = *HSTU_LDS(const vec8, kt + (o % NS) * 32 * KROW + kaddr[4 * (o / NS) + j]);
                    }
                }
            };
#pragma unroll
            for (int sub = 0; sub < NS; ++sub)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[sub][r] = 0.f;
            vec8 fa[2][4];
            load_group(0, fa[0]);
#pragma unroll
            for (int m = 0; m < NOPS; ++m) {
                __builtin_amdgcn_sched_barrier(0);
                if (m + 1 < NOPS) load_group(m + 1, fa[(m + 1) & 1]);
                const int o = m >> 1;
                if ((m & 1) == 0) {
                    vec8 b[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) b[j] = pb[j >> 1][j & 1];
                    oacc[o][0] = TT::mfma64(fa[m & 1], b, oacc[o][0]);
                } else {
                    vec8 b[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) b[j] = qreg[4 * (o / NS) + j];
                    s[o % NS] = TT::mfma64(fa[m & 1], b, s[o % NS]);
                }
                if (m % (NOPS / NPW) == (NOPS / NPW) - 1) issue_copy(slot_c, m / (NOPS / NPW));
            }
            __builtin_amdgcn_sched_barrier(0);
            return;
        }
        auto load_op = [&](int k) __attribute__((always_inline)) -> vec8 {
            const int o = k >> 1;
            if ((k & 1) == 0) {
                const int sub = o / (2 * DT), tt = (o / DT) % 2, dt = o % DT;
                const char* vb = vt + (sub * 32 + tt * 16) * VROW;
                return read_vt_operand<TT>(vb + vaddr[0][dt], vb + vaddr[0][dt] + 8 * VROW);
            } else {
                const int ks = o / NS, sub = o % NS;
                return *HSTU_LDS(const vec8, kt + sub * 32 * KROW + kaddr[ks]);
            }
        };
#pragma unroll
        for (int sub = 0; sub < NS; ++sub)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[sub][r] = 0.f;
        vec8 fr[PD];
#pragma unroll
        for (int k = 0; k < PD; ++k) fr[k] = load_op(k);
#pragma unroll
        for (int k = 0; k < NOPS; ++k) {
            __builtin_amdgcn_sched_barrier(0);
            const int o = k >> 1;
            if ((k & 1) == 0) {
                const int sub = o / (2 * DT), tt = (o / DT) % 2, dt = o % DT;
                oacc[dt][0] = TT::mfma(fr[k % PD], pb[sub][tt], oacc[dt][0]);
            } else {
                const int ks = o / NS, sub = o % NS;
                s[sub] = TT::mfma(fr[k % PD], qreg[ks], s[sub]);
            }
            if (k + PD < NOPS) fr[k % PD] = load_op(k + PD);
            // spread the copies over the phase: one after every (NOPS/NPW)-th MFMA
            if (k % (NOPS / NPW) == 1) issue_copy(slot_c, k / (NOPS / NPW));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // VALU phase: P^T from S^T of `tile`.
    auto valu_phase = [&](int tile) __attribute__((always_inline)) {
        if (tile >= full_begin && tile < full_end) {
#pragma unroll
            for (int sub = 0; sub < NS; ++sub) silu_pack<TT, 0>(s[sub], pb[sub], p.c1, M, row, 0);
        } else if (plain_causal) {
#pragma unroll
            for (int sub = 0; sub < NS; ++sub) silu_pack<TT, 2>(s[sub], pb[sub], p.c1, M, row, tile * BN + 4 * g + sub * 32);
        } else {
#pragma unroll
            for (int sub = 0; sub < NS; ++sub) silu_pack<TT, 1>(s[sub], pb[sub], p.c1, M, row, tile * BN + 4 * g + sub * 32);
        }
    };
    auto end_of_step = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): every copy has landed for this wave ...
        __syncthreads();                     // ... and for every wave
    };
    typedef std::integral_constant<int, 0> S0;
    typedef std::integral_constant<int, 1> S1;

    // Step i uses slot i % 2; step 0 is peeled (first product only), then whole rounds of two steps, then the
    // remainder.  [matrix(i) | VALU(i)] per step, one barrier at its end.
    const int rounds = (T - 1) / NSLOT, rem = (T - 1) % NSLOT;
    auto step = [&](auto slot_c) __attribute__((always_inline)) {
        __builtin_amdgcn_s_setprio(3);  // the matrix core must not wait behind the VALU work of the CU's other workgroup
        matrix_phase(slot_c);
        __builtin_amdgcn_s_setprio(0);
        valu_phase(t_cur);
        end_of_step();
        ++t_cur;
    };
    gemm1_only(0);
    valu_phase(t_cur);
    end_of_step();
    ++t_cur;
    for (int r = 0; r < rounds; ++r) {
        step(S1{});
        step(S0{});
    }
    if (rem >= 1) step(S1{});
    gemm2_only((T - 1) % NSLOT);
    // the redundant copies of the last steps may still be in flight: they must land before the LDS is released
    __builtin_amdgcn_s_waitcnt(0x0F70);

    if (my_partial) {
        store_partial<DT>(oacc, 0, my_partial, orow0, wq0 + l32, nq, p.H, W.h, g);
        if (W.split == 0 && threadIdx.x == 0) p.split_counts[W.block_id] = W.nsplit;
    } else if constexpr (4 * 32 * (DT * 64 + 16) <= NSLOT * (KTILE + VTILE)) {
        // the K/V tiles are dead once every wave is through its last product; each wave then turns its output
        // tile around in its own piece of that LDS
        __syncthreads();
        store_output_via_lds<TT, DT>(oacc, smem + wave * (32 * (DT * 64 + 16)), p.o, orow0, wq0, nq, p.o_rs, p.o_hs, W.h,
                                     lane, output_scale(p, orow0 + (wq0 + l32 < nq ? wq0 + l32 : nq - 1)));
    } else {
        // 8-bit K/V tiles are smaller than the 16-bit output staging would be
        store_output<TT, DT>(oacc, 0, p.o, orow0, wq0 + l32, nq, p.o_rs, p.o_hs, W.h, g,
                             output_scale(p, orow0 + (wq0 + l32 < nq ? wq0 + l32 : nq - 1)));
    }
    };  // process_item
    int parity = 0;  // two hand-over words used in turn: a wave may still be reading one when thread 0, an item
                     // without barriers later, writes the next
    int victim = xcd;           // whose list thread 0 draws from ...
    int limit = slots_per_xcd;  // ... and how many items that list holds
    while (bid >= 0) {
        int ticket = 0;  // per lane; only thread 0's is meaningful
        int next = -1;   // wave-uniform
        if (queue) {
            if (threadIdx.x == 0) ticket = atomicAdd(queue + victim * 16, 1);
        } else {
            ++round;
            const int ns = round * GL + ((round & 1) ? GL - 1 - lw : lw);
            if (ns < slots_per_xcd) next = ns * 8 + xcd;
        }
        process_item();
        if (queue) {
            if (threadIdx.x == 0) {
                int nb = -1;
                for (int tries = 0;;) {
                    if (ticket < limit) {
                        nb = ticket * 8 + victim;
                        break;
                    }
                    if (++tries == 8) break;  // every list is exhausted
                    victim = (victim + 1) & 7;
                    if (p_arg.nitems) limit = p_arg.nitems[victim];
                    ticket = atomicAdd(queue + victim * 16, 1);
                }
                *HSTU_LDS(int, smem + NEXT_OFF + parity * 4) = nb;
            }
            __syncthreads();  // hands over the next item, and every wave is done with the LDS tiles of this one
            next = *HSTU_LDS(const int, smem + NEXT_OFF + parity * 4);
            parity ^= 1;
        } else {
            __syncthreads();  // every wave is done with the LDS tiles before the next item's first copies land
        }
        bid = __builtin_amdgcn_readfirstlane(next);
    }
}

}  // namespace hstu
