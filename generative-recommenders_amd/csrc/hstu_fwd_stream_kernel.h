// Streaming two-group forward kernel for long sequences (tile config 2): 8 waves per workgroup, 256 query rows, one
// persistent workgroup per CU, a ring of three K and three V tiles in LDS.
//
// The matrix cores and the pointwise s*sigmoid(alpha s) cost the same issue time per score, and a wave that has just
// issued an MFMA cannot issue VALU work for a while (hstu_fwd_pp_kernel.h), so the two kinds of work come from different
// waves of a SIMD at the same time: waves 0-3 ("A") run [matrix phase of tile i | VALU phase of tile i] while waves
// 4-7 ("B"), which share their SIMDs, run [VALU phase of tile i-1 | matrix phase of tile i] -- half a step apart, held
// there by one barrier per step.  The matrix phase interleaves O^T += V^T P^T of the previous tile with S^T = K Q^T of
// this one; in step i the A waves issue the copies of V(i+1) and K(i+2) from inside it (their slots were last read in
// step i-1), and the end of step i waits only for the copies issued in step i-1.
//
// "Streaming": work items follow each other without the pipeline running empty in between.
//
// What an item costs besides its steps is latency, not work: its Q rows are the one thing nobody has touched yet (a
// cold read from HBM), its first tiles have to come in before the first product, its output has to be turned around and
// stored.  Here all of that lies in the shadow of the neighbouring items:
//  * The id of the next item is known after the first step of the current one (strided deal: arithmetic; counters: one
//    thread of a wave that idles in that step anyway draws the ticket and hands the id over through LDS).
//  * When the last step of an item ends, the K slots are dead and no copy is in flight.  Every wave then decodes the next
//    item and starts a copy of ITS 32 rows of the next Q into an LDS area of its own, laid out like a K tile (whole rows,
//    16 bytes per lane: a wave that loads the operand layout directly asks for 32 bytes of 32 different rows with every
//    instruction, and the eight waves together then keep the vector memory path busy for thousands of cycles), and the
//    copy waves start the next item's first tiles (K into slots 0 and 1, V into slot 0 unless the drain still reads that
//    slot: then it follows after the hand-over barrier, a full step before its first use).  Only then comes the drain:
//    the last P^T, the last second product, the output.  The copies have the length of the drain to arrive.
//  * The output is turned around in ring slots that neither the drain nor the next item's first tiles use (4 KB per wave,
//    two passes of 128-byte row pieces), or in LDS of its own where the ring is small, so no barrier separates it from
//    the ring's last readers or from the next item's first copies: the two groups drain side by side and meet again at
//    the one barrier that opens the next item.
// Per item: T + 2 barriers, none of them a fence (output stores stay in flight across them; what a barrier has to order
// is awaited explicitly in front of it).
#pragma once
#include "hstu_fwd_pp_kernel.h"

namespace hstu {

// Row-contiguous store of a wave's 32 x DV output tile (16-bit elements) through `stage`, LDS that only this wave
// touches: per pass the lanes write SRB = 128 (64 for dv = 32) bytes of every row in accumulator layout -- 16-byte chunks
// XOR-ed with the row number as in a K tile, so that neither side meets a bank twice -- and read them back 16 bytes per
// lane, 8 (16) rows per store instruction.  BLOCKED: the 32 staged rows are four blocks of 1 KB that lie 4 KB apart
// (the blocks of a tile slot that the wave's own copy instructions write); otherwise they are contiguous.
template <class TT, int DT, bool BLOCKED>
__device__ __forceinline__ void store_output_staged(const f32x16_t (&oacc)[DT][1], char* stage, char* o, int64_t orow0, int q0, int nq,
                                                    int64_t o_rs, int64_t o_hs, int h, int lane, float oscale) {
    typedef typename TT::out_elem elem;  // 16 bits
    typedef __attribute__((ext_vector_type(4))) elem elem4;
    constexpr int SDT = DT >= 2 ? 2 : 1;  // dv tiles per pass
    constexpr int SRB = SDT * 64;         // bytes of a row per pass
    constexpr int CH = SRB / 16;          // 16-byte chunks of that
    constexpr int RPI = 64 / CH;          // rows per store instruction
    static_assert(!BLOCKED || SRB == 128, "a 1 KB block holds 8 staged rows");
    auto row_at = [&](int j) -> int { return BLOCKED ? (j >> 3) * 4096 + (j & 7) * 128 : j * SRB; };
    const int l32 = lane & 31, g = lane >> 5;
    const int chunk = lane % CH, rsub = lane / CH;
    char* op = o + ((orow0 + q0 + rsub) * o_rs + (int64_t)h * o_hs) * 2 + chunk * 16;
#pragma unroll
    for (int pass = 0; pass < DT / SDT; ++pass) {
#pragma unroll
        for (int dl = 0; dl < SDT; ++dl)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                elem4 o4;
#pragma unroll
                for (int i = 0; i < 4; ++i) o4[i] = (elem)(oacc[pass * SDT + dl][0][r4 * 4 + i] * oscale);
                *HSTU_LDS(elem4, stage + row_at(l32) + (((dl * 4 + r4) ^ swz_k<CH>(l32)) * 16) + g * 8) = o4;
            }
#pragma unroll
        for (int i = 0; i < 32 / RPI; ++i) {
            const int row = i * RPI + rsub;
            const i32x4_t v = *HSTU_LDS(const i32x4_t, stage + row_at(row) + ((chunk ^ swz_k<CH>(row)) * 16));
            if (q0 + row < nq) *(i32x4_t*)(op + (int64_t)i * RPI * o_rs * 2 + pass * SRB) = v;
        }
    }
}

template <class TT, int DQK, int DV, int BN>
__global__ __launch_bounds__(512, 2) void hstu_fwd_stream_kernel(const FwdParams p_arg) {
    typedef typename TT::vec8 vec8;
    static_assert(DQK == DV, "the interleaved matrix phase assumes as many first-product as second-product MFMAs");
    constexpr int BM = 256;
    constexpr int NS = BN / 32;
    constexpr int KS = DQK / 16;
    constexpr int DT = DV / 32;
    constexpr int ES = TT::ES;
    constexpr int KROW = DQK * ES, VROW = DV * ES;
    constexpr int KTILE = BN * KROW, VTILE = BN * VROW;
    constexpr int NSLOT = 3;
    constexpr int RING = NSLOT * (KTILE + VTILE);
    constexpr int QSTAGE_W = 32 * KROW;                 // per wave: its rows of the next Q
    constexpr int QSTAGE_OFF = RING;
    constexpr int STAGE_W = 32 * (DT >= 2 ? 128 : 64);  // per wave: output staging
    // The output is staged in LDS of its own where that fits; otherwise in the ring: waves 0-3 in K slot 2, waves 4-7 in
    // a V slot that neither the drain reads nor the next item's first V tile is copied to.
    constexpr bool OUT_IN_RING = RING + 8 * QSTAGE_W + 8 * STAGE_W > 160 * 1024;
    constexpr int STAGE_OFF = QSTAGE_OFF + 8 * QSTAGE_W;
    static_assert(!OUT_IN_RING || (4 * STAGE_W <= KTILE && 4 * STAGE_W <= VTILE), "output staging in ring slots");
    // The next item's id travels from the drawing thread to every wave through the first word of that wave's Q area,
    // which nothing else touches between the wave's read of its Q rows and its next copy into it.
    // The ring is the first LDS object (address 0), so that every tile and slot offset folds into the immediate field
    // of the LDS reads.
    __shared__ __attribute__((aligned(1024))) char smem[STAGE_OFF + (OUT_IN_RING ? 0 : 8 * STAGE_W)];
    constexpr int VOFF = NSLOT * KTILE;
    constexpr int VBIAS = (RING > 65536) ? 32768 : 0;
    static_assert(VOFF >= VBIAS && VOFF - VBIAS + NSLOT * VTILE <= 65536 && NSLOT * KTILE <= 65536, "LDS immediates");
    constexpr bool WIDE = ES == 1 && DQK % 64 == 0 && BN == 64;
    constexpr int NOPS = WIDE ? (NS * KS + NS * 2 * DT) / 4 : NS * KS + NS * 2 * DT;  // MFMAs of one matrix phase
    constexpr int PD = NOPS >= 16 ? 6 : 4;                                          // operands in flight (16-deep scheme)

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = wave >> 2;  // 0: waves 0-3 (A), 1: waves 4-7 (B); waves w and w+4 share a SIMD
    const int g = lane >> 5;
    const int l32 = lane & 31;

    // Item ids are slot * 8 + xcd (see hstu_fwd_pp_kernel.h): dealt with a stride in alternating direction, or drawn from
    // the per-XCD counters, own list first.
    const int GL = gridDim.x >> 3, lw = blockIdx.x >> 3, xcd = blockIdx.x & 7;
    const int slots_per_xcd = p_arg.nitems ? HSTU_CONST(int, p_arg.nitems)[xcd] : p_arg.slots_per_xcd;
    int* const queue = p_arg.queue;
    int round = 0;
    int parity = 0;
    int victim = xcd;           // whose list the drawing wave draws from ...
    int limit = slots_per_xcd;  // ... and how many items that list holds
    const bool drawer = wave == 4;  // this wave waits for the other group in every first step anyway; its lane 0 talks to memory

    typedef TileCopy<BN, KROW, false, ES> KCopy;
    typedef TileCopy<BN, VROW, true, ES> VCopy;
    constexpr int NPW = KCopy::PER_WAVE + VCopy::PER_WAVE;  // copy instructions per wave and step
    static_assert(NPW <= 15 && NOPS % NPW == 0, "vmcnt immediate / even spread of the copies");

    // ---- the item in progress: what its steps, its drain and its output need -------------------------------------
    SeqMask M;
    RowMask row;
    int n = 0, nq = 0, wq0 = 0, h_cur = 0, full_begin = 0, full_end = 0, jt_end = 0, T = 0, t_cur = 0;
    int split = 0, nsplit = 0, block_id = 0;
    int drain_slot = 0;  // (T - 1) % 3: the slot of the item's last tile, which the drain reads
    bool plain_causal = false;
    int64_t orow0 = 0;
    float* my_partial = nullptr;
    i32x4_t kbase = {0, 0, 0, 0}, vbase = {0, 0, 0, 0};  // (copy waves) descriptors of the sequence's K and V rows for this head
    unsigned k_rsb = 0, v_rsb = 0;
    float c1 = 0.f;
    KCopy kcopy;
    VCopy vcopy;
    vec8 qreg[KS];
    int kaddr[KS];
    int vaddr[2][DT];
    f32x16_t oacc[DT][1];
    f32x16_t s[NS];   // S^T of the tile in flight between this wave's matrix and VALU phases
    vec8 pb[NS][2];   // P^T of the tile in flight between its VALU phase and its next matrix phase

    // ---- building blocks (as in hstu_fwd_pp_kernel.h) --------------------------------------------------------------
    typedef std::integral_constant<int, 0> S0;
    typedef std::integral_constant<int, 1> S1;
    typedef std::integral_constant<int, 2> S2;
    // Copy instruction j (0 .. NPW-1) of the step of list entry i (SLOT = i % 3): the V tile of entry i + 1, then the K
    // tile of entry i + 2.  Past the end of the list the LAST entry is copied again, into the slot it already lives in
    // (slot `drain_slot`): the same bytes over themselves, which disturbs no reader, keeps the number of copy instructions
    // per step (and with it the vmcnt arithmetic) constant, and leaves every other slot quiet for the drain.
    auto issue_copy = [&](auto slot_c, int j) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        if (grp != 0) return;
        if (j < VCopy::PER_WAVE) {
            const bool past = t_cur + 1 >= jt_end;
            vcopy.issue_one(j, vbase, v_rsb, (past ? jt_end - 1 : t_cur + 1) * BN,
                            smem + VOFF + (past ? drain_slot : (SLOT + 1) % NSLOT) * VTILE, wave);
        } else {
            const bool past = t_cur + 2 >= jt_end;
            kcopy.issue_one(j - VCopy::PER_WAVE, kbase, k_rsb, (past ? jt_end - 1 : t_cur + 2) * BN,
                            smem + (past ? drain_slot : (SLOT + 2) % NSLOT) * KTILE, wave);
        }
    };
    // S^T = K Q^T only (first step; K slot 0).  COPIES: this wave's share of the step's copies goes out between the MFMAs.
    auto gemm1_only = [&](auto copies_c) __attribute__((always_inline)) {
        constexpr bool COPIES = decltype(copies_c)::value;
        constexpr int NM = WIDE ? NS * KS / 4 : NS * KS;  // MFMAs
        const char* kt = smem;
        int m = 0;
#pragma unroll
        for (int sub = 0; sub < NS; ++sub) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[sub][r] = 0.f;
#pragma unroll
            for (int kk = 0; kk < (WIDE ? KS / 4 : KS); ++kk, ++m) {
                if constexpr (WIDE) {
                    vec8 a[4], b[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        a[j] = *HSTU_LDS(const vec8, kt + sub * 32 * KROW + kaddr[4 * kk + j]);
                        b[j] = qreg[4 * kk + j];
                    }
                    s[sub] = TT::mfma64(a, b, s[sub]);
                } else {
                    vec8 a = *HSTU_LDS(const vec8, kt + sub * 32 * KROW + kaddr[kk]);
                    s[sub] = TT::mfma(a, qreg[kk], s[sub]);
                }
                if constexpr (COPIES) {
#pragma unroll
                    for (int j = m * NPW / NM; j < (m + 1) * NPW / NM; ++j) issue_copy(S0{}, j);
                }
            }
        }
    };
    auto gemm2_only = [&](int vslot) __attribute__((always_inline)) {
        const char* vt = smem + (VOFF - VBIAS) + vslot * VTILE;
        if constexpr (WIDE) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                vec8 a[4], b[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
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
    auto matrix_phase = [&](auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        const char* kt = smem + SLOT * KTILE;
        const char* vt = smem + (VOFF - VBIAS) + ((SLOT + NSLOT - 1) % NSLOT) * VTILE;
        if constexpr (WIDE) {
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
        // MFMA k: even k -> second product (sub, tt, dt) = ((k/2)/(2 DT), ((k/2)/DT) % 2, (k/2) % DT);
        //         odd k  -> first product  (ks, sub) = ((k/2)/NS, (k/2) % NS).
        // (Measured equal or slightly slower: one product after the other, and each accumulator's MFMAs in a row.)
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
            if (k % (NOPS / NPW) == 1) issue_copy(slot_c, k / (NOPS / NPW));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto valu_phase = [&](int tile) __attribute__((always_inline)) {
        if (tile >= full_begin && tile < full_end) {
#pragma unroll
            for (int sub = 0; sub < NS; ++sub) silu_pack<TT, 0>(s[sub], pb[sub], c1, M, row, 0);
        } else if (plain_causal) {
#pragma unroll
            for (int sub = 0; sub < NS; ++sub) silu_pack<TT, 2>(s[sub], pb[sub], c1, M, row, tile * BN + 4 * g + sub * 32);
        } else {
#pragma unroll
            for (int sub = 0; sub < NS; ++sub) silu_pack<TT, 1>(s[sub], pb[sub], c1, M, row, tile * BN + 4 * g + sub * 32);
        }
    };
    // A plain s_barrier: no fence, so loads and stores the compiler knows of stay in flight across it.
    auto bar = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    auto end_of_step = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt((NPW & 0xF) | ((NPW >> 4) << 14) | 0x0F70);  // every copy but this step's has landed for this wave ...
        bar();                                                                   // ... and for every wave
    };
    // The drawing wave (everything wave-uniform): a ticket from the list of `victim` ...
    auto ask_ticket = [&]() __attribute__((always_inline)) -> int {  // lane 0's value; not waited for
        int t = 0;
        if (lane == 0) t = atomicAdd(queue + victim * 16, 1);
        return t;
    };
    auto draw_ticket = [&]() __attribute__((always_inline)) -> int { return __builtin_amdgcn_readfirstlane(ask_ticket()); };
    // ... and the next item from the ticket it holds (own list first, then the other XCDs').
    auto resolve_ticket = [&](int ticket) __attribute__((always_inline)) -> int {
        int nb = -1;
        for (int tries = 0;;) {
            if (ticket < limit) {
                nb = ticket * 8 + victim;
                break;
            }
            if (++tries == 8) break;  // every list is exhausted
            victim = (victim + 1) & 7;
            if (p_arg.nitems) limit = HSTU_CONST(int, p_arg.nitems)[victim];
            ticket = draw_ticket();
        }
        return nb;
    };
    // Every wave, after the barrier that follows the drawing thread's write (counters), or on its own (strided deal).
    auto publish_next = [&](int nb) __attribute__((always_inline)) {  // the drawing wave
        if (lane == 0) {
#pragma unroll
            for (int w = 0; w < 8; ++w) *HSTU_LDS(int, smem + QSTAGE_OFF + w * QSTAGE_W + parity * 4) = nb;
        }
    };
    auto collect_next = [&]() __attribute__((always_inline)) -> int {
        int next = -1;
        if (queue) {
            next = *HSTU_LDS(const int, smem + QSTAGE_OFF + wave * QSTAGE_W + parity * 4);
            parity ^= 1;
        } else {
            ++round;
            const int ns = round * GL + ((round & 1) ? GL - 1 - lw : lw);
            if (ns < slots_per_xcd) next = ns * 8 + xcd;
        }
        return __builtin_amdgcn_readfirstlane(next);
    };

    int next_bid = lw < slots_per_xcd ? lw * 8 + xcd : -1;
    bool v0_late = false;  // the next item's first V tile could not be copied during the drain: it follows after the hand-over

    // The parameters are read from the kernel argument segment again wherever they are needed (scalar loads that hit
    // the scalar cache): held in registers across the item loop they would not fit the scalar register file.
    auto params = [&]() __attribute__((always_inline)) -> const FwdParams& {
        const __attribute__((address_space(4))) FwdParams* pk =
            (const __attribute__((address_space(4))) FwdParams*)__builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("" : "+s"(pk));
        return *(const FwdParams*)pk;
    };
    // Decodes item `next_bid`; an item without work (a row block past the end of a short sequence, a run of a kv split
    // that a short range does not reach) only hands the next id over.  False: nothing is left.
    auto find_next = [&](const FwdParams& p, Work& W) __attribute__((always_inline)) -> bool {
        for (;;) {
            if (next_bid < 0) return false;
            if (decode_work<BM, BN>(W, next_bid) && W.jt_end > W.jt_begin) return true;
            if (queue) {
                if (drawer) publish_next(resolve_ticket(draw_ticket()));
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
                bar();
            }
            next_bid = collect_next();
        }
    };
    // Starts the copies of this wave's rows of the item's Q and (copy waves) of its first tiles: K into slots 0 and 1, V
    // into slot 0 unless the drain of the item in progress still reads that slot.
    auto prefetch = [&](const FwdParams& p, const Work& W, int lane_v, auto grp_c) __attribute__((always_inline)) {
        const int64_t qrow0 = p.delta > 0 ? (int64_t)W.b * p.delta : W.seq_start;
        const unsigned q_rsb = (unsigned)p.q_rs * ES;
        copy_q_rows<KROW>(make_buffer_rsrc(p.q + (qrow0 * p.q_rs + (int64_t)W.h * p.q_hs) * ES, (unsigned)W.nq * q_rsb), q_rsb,
                          W.m0 + wave * 32, smem + QSTAGE_OFF + wave * QSTAGE_W, lane_v);
        if constexpr (decltype(grp_c)::value == 0) {
            // descriptors of the sequence's K and V rows for this head (the host keeps rows * stride below 2^32)
            k_rsb = (unsigned)p.k_rs * ES;
            v_rsb = (unsigned)p.v_rs * ES;
            kbase = make_buffer_rsrc(p.k + (W.seq_start * p.k_rs + (int64_t)W.h * p.k_hs) * ES, (unsigned)W.n * k_rsb);
            vbase = make_buffer_rsrc(p.v + (W.seq_start * p.v_rs + (int64_t)W.h * p.v_hs) * ES, (unsigned)W.n * v_rsb);
            kcopy.init(wave, lane_v, k_rsb);
            vcopy.init(wave, lane_v, v_rsb);
            const int t0 = W.jt_begin, t1 = t0 + 1 < W.jt_end ? t0 + 1 : t0;
            kcopy.issue(kbase, k_rsb, t0 * BN, smem, wave);
            if (!v0_late) vcopy.issue(vbase, v_rsb, t0 * BN, smem + VOFF, wave);
            kcopy.issue(kbase, k_rsb, t1 * BN, smem + KTILE, wave);
        }
    };
    // Everything this wave has asked for is awaited: its Q rows, its share of the first tiles (and the output stores of
    // the item before).  The Q operand is read with the offsets of the first 32 rows of a K tile.
    auto take_q = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qreg[ks] = *HSTU_LDS(const vec8, smem + QSTAGE_OFF + wave * QSTAGE_W + kaddr[ks]);
        prescale_q<TT, KS>(qreg, c1);
    };
    // The decoded item becomes the item in progress: mask ranges, addresses, zeroed accumulators, Q in operand form.
    auto adopt = [&](const FwdParams& p, const Work& W, int lane_v, bool with_q) __attribute__((always_inline)) {
        M = W.M;
        n = W.n;
        nq = W.m1;  // one past the last row of this item: rows from here on are never loaded or stored
        wq0 = W.m0 + wave * 32;
        h_cur = W.h;
        split = W.split;
        nsplit = W.nsplit;
        block_id = W.block_id;
        c1 = p.c1;
        const int wR0 = W.rbase + wq0;
        const int wR1 = (wq0 + 32 < nq ? W.rbase + wq0 + 32 : W.rbase + nq) - 1;
        // Tiles [full_begin, full_end) are valid in every element for this wave's rows (no mask code); see
        // hstu_fwd_pp_kernel.h.
        full_begin = 0;
        full_end = 0;
        if (wR1 >= wR0 && W.u >= p.c && W.u >= 0) {
            const int idr_lo = M.id(wR0), idr_hi = M.id(wR1);
            full_end = (idr_lo + M.shift) / BN;
            if (full_end * BN > n) full_end = n / BN;
            if (p.w > 0 && idr_hi - p.w > 0) full_begin = (idr_hi - p.w + M.shift + BN - 1) / BN;
        }
        plain_causal = p.w == 0 && p.c == 0 && p.targets == nullptr;
        jt_end = W.jt_end;
        T = jt_end - W.jt_begin;
        drain_slot = (T - 1) % NSLOT;
        t_cur = W.jt_begin;
        orow0 = p.delta > 0 ? (int64_t)W.b * p.delta : W.seq_start;
        my_partial = p.kv_splits > 1 ? p.partial + (int64_t)W.split * p.partial_stride : nullptr;
        row.init(M, wR0 + l32);
        lds_read_offsets<TT, DQK, DV>(kaddr, vaddr, lane_v);
        // (only vaddr[0] is kept: the second transposing read of an operand lies 8 rows below the first for every lane,
        // which is an immediate)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            vaddr[0][dt] += VBIAS;
            asm volatile("" : "+v"(vaddr[0][dt]));  // keep the bias in the register, out of the immediates
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][0][r] = 0.f;
        if (with_q) take_q();
    };
    // `more`: the copies of a next item have been started.
    auto store_item = [&](const FwdParams& p, bool more) __attribute__((always_inline)) {
        if (my_partial) {
            store_partial<DT>(oacc, 0, my_partial, orow0, wq0 + l32, nq, p.H, h_cur, g);
            if (split == 0 && threadIdx.x == 0) p.split_counts[block_id] = nsplit;
            return;
        }
        const float osc = output_scale(p, orow0 + (wq0 + l32 < nq ? wq0 + l32 : nq - 1));
        if constexpr (OUT_IN_RING) {
            // Waves 0-3 stage in K slot 2, each in the four 1 KB blocks that its own copy instructions write: the only
            // copies that can still be in flight into that slot are the wave's own of the last step (when the last tile
            // lives there), so the wave waits for them itself -- they are older than the copies it has just started for
            // the next item, whose number it knows.  Waves 4-7 stage in a V slot that neither the drain reads nor the
            // last step copied to nor the next item's first V tile goes to: slot 2 if the drain reads slot 1, else slot 1.
            char* stage;
            if (grp == 0) {
                constexpr int NQ = 32 * KROW / 1024, NK = 2 * KCopy::PER_WAVE, NV = VCopy::PER_WAVE;
                if (!more)
                    __builtin_amdgcn_s_waitcnt(0x0F70);
                else if (v0_late)
                    __builtin_amdgcn_s_waitcnt(((NQ + NK) & 0xF) | (((NQ + NK) >> 4) << 14) | 0x0F70);
                else
                    __builtin_amdgcn_s_waitcnt(((NQ + NK + NV) & 0xF) | (((NQ + NK + NV) >> 4) << 14) | 0x0F70);
                stage = smem + 2 * KTILE + (wave & 3) * 1024;
            } else {
                stage = smem + VOFF + (drain_slot == 1 ? 2 : 1) * VTILE + (wave & 3) * 1024;
            }
            store_output_staged<TT, DT, true>(oacc, stage, p.o, orow0, wq0, nq, p.o_rs, p.o_hs, h_cur, lane, osc);
        } else {
            store_output_staged<TT, DT, false>(oacc, smem + STAGE_OFF + wave * STAGE_W, p.o, orow0, wq0, nq, p.o_rs, p.o_hs, h_cur, lane, osc);
        }
    };
    // Per-lane values that depend on the lane number only are recomputed for every item: hoisted out of the item loop
    // they would be spilled.  The empty asm hides from the compiler that the lane number is the same every time.
    auto lane_again = [&]() __attribute__((always_inline)) -> int {
        int lane_v = lane;
        asm volatile("" : "+v"(lane_v));
        return lane_v;
    };

    // The two groups run the same item loop, each with its own order of phases; they meet at the barriers, which both
    // execute in the same number: one that opens an item, one in its first step, one at the end of every step.
    if (grp == 0) {
        // ---- A: [matrix(i) | VALU(i)] per step
        typedef std::integral_constant<int, 0> G;
        auto stepA = [&](auto slot_c) __attribute__((always_inline)) {
            __builtin_amdgcn_s_setprio(3);  // the matrix core must not wait behind the other wave's VALU work
            matrix_phase(slot_c);
            __builtin_amdgcn_s_setprio(0);
            valu_phase(t_cur);
            end_of_step();
            ++t_cur;
        };
        Work W;
        bool more = find_next(params(), W);
        if (more) prefetch(params(), W, lane_again(), G{});
        while (more) {
            adopt(params(), W, lane_again(), true);
            bar();  // the item's first tiles are in LDS for every wave, and nobody reads the previous item's any more
            if (v0_late) vcopy.issue(vbase, v_rsb, t_cur * BN, smem + VOFF, wave);
            gemm1_only(std::true_type{});
            bar();
            valu_phase(t_cur);
            end_of_step();
            next_bid = collect_next();
            ++t_cur;
            const int rounds = (T - 1) / NSLOT, rem = (T - 1) % NSLOT;
            for (int r = 0; r < rounds; ++r) {
                stepA(S1{});
                stepA(S2{});
                stepA(S0{});
            }
            if (rem >= 1) stepA(S1{});
            if (rem >= 2) stepA(S2{});
            // The K slots are dead: the next item's copies go out ahead of the output.  (The last second product first:
            // the other group starts its copies of the next Q rows now, and the vector memory path takes one 1 KB copy
            // per 16 cycles -- this group's 20 per wave would only stand in their way, while it has time to spare.)
            more = find_next(params(), W);
            v0_late = rem == 0;  // the drain reads V slot (T - 1) % 3
            gemm2_only(rem);
            if (more) prefetch(params(), W, lane_again(), G{});
            store_item(params(), more);
        }
    } else {
        // ---- B: [VALU(i-1) | matrix(i)] per step, one phase behind A
        typedef std::integral_constant<int, 1> G;
        auto stepB = [&](auto slot_c) __attribute__((always_inline)) {
            valu_phase(t_cur - 1);
            __builtin_amdgcn_s_setprio(3);
            matrix_phase(slot_c);
            __builtin_amdgcn_s_setprio(0);
            end_of_step();
            ++t_cur;
        };
        Work W;
        bool more = find_next(params(), W);
        if (more) prefetch(params(), W, lane_again(), G{});
        while (more) {
            adopt(params(), W, lane_again(), false);
            bar();
            // this group waits for the other one's first product anyway: its Q rows are taken (and the ticket drawn) now
            take_q();
            int ticket = 0;  // only lane 0 of the drawing wave holds one; asked for now, looked at after the first product
            if (queue && drawer) ticket = ask_ticket();
            bar();
            gemm1_only(std::false_type{});
            if (queue && drawer) {
                publish_next(resolve_ticket(__builtin_amdgcn_readfirstlane(ticket)));
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the words are written before the barrier
            }
            end_of_step();
            next_bid = collect_next();
            ++t_cur;
            const int rounds = (T - 1) / NSLOT, rem = (T - 1) % NSLOT;
            for (int r = 0; r < rounds; ++r) {
                stepB(S1{});
                stepB(S2{});
                stepB(S0{});
            }
            if (rem >= 1) stepB(S1{});
            if (rem >= 2) stepB(S2{});
            more = find_next(params(), W);
            if (more) prefetch(params(), W, lane_again(), G{});
            valu_phase(t_cur - 1);
            gemm2_only(rem);
            store_item(params(), more);
        }
    }
    // the redundant copies of the last steps may still be in flight: they must land before the LDS is released
    __builtin_amdgcn_s_waitcnt(0x0F70);
}

}  // namespace hstu
