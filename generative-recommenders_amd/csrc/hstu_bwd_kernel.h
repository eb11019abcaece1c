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
// Kernels, none with atomics, so the result does not depend on the schedule:
//   * hstu_bwd_dkdv_kernel: a workgroup owns 128 key rows (K and V of 32 rows per wave in registers, K pre-scaled
//     by c1 = -alpha * log2(e)) and walks the query rows that can see them in tiles of 64 (Q and dOut through LDS):
//         S[q, kv]   = Q K^T          A = Q tile (row reads),            B = K registers
//         dP[q, kv]  = dOut V^T       A = dOut tile (row reads),         B = V registers
//         dV^T[dv, kv] += dOut^T P    A = dOut tile (transposing reads), B = P packed from the accumulator
//         dK^T[d, kv]  += Q^T dS      A = Q tile (transposing reads),    B = dS packed
//     On request it also writes every block of dS to scratch memory.
//   * hstu_bwd_dq_kernel: a workgroup owns 128 query rows (Q pre-scaled and dOut in registers) and walks the key
//     rows as the forward kernel does:
//         S^T[kv, q]  = K Q^T         A = K tile (row reads),            B = Q registers
//         dP^T[kv, q] = V dOut^T      A = V tile (row reads),            B = dOut registers
//         dQ^T[d, q] += K^T dS^T      A = K tile (transposing reads),    B = dS^T packed
//   * hstu_bwd_dq_stored_kernel, instead of the former when dS was stored: only the last of these three products, with
//     dS^T read back from the scratch memory.
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
    // Stored-dS mode (both null / 0 otherwise): the key-stationary kernel writes every block of dS it forms, rounded
    // to the operand type, and hstu_bwd_dq_stored_kernel reads them back instead of forming S and dP again.
    char* ds;
    int ds_pitch32;  // blocks of 32 keys per row of blocks: 4 * ceil(max_seq_len / 128)
};

// Where the dS blocks of one (sequence, head) pair live.  A block is 32 query rows x 32 keys, 2 KB, in the register
// image of the wave that formed it: half h (query rows 16 h ..), lane (key c = lane % 32, g = lane / 32) holds 16 bytes
// = query rows 16 h + 8 j + 4 g + {0..3}, j = 0, 1, at 16-byte position 64 h + ((2 c + g) ^ 8 h) -- every store covers
// a contiguous KB, and the XOR makes the transposing LDS reads of the consumer conflict-free.  Sequence b owns the
// bytes of (len_b + 32) rows x H x pitch32 x 64, enough for H x ceil(len_b / 32) x pitch32 blocks, starting at
// (offset_b + 32 b) rows; block (h, qb, kb) is number (h * nqb + qb) * pitch32 + kb of them.
__device__ __forceinline__ char* ds_pair_base(const BwdParams& bp, const Work& W, int n) {
    const int64_t row_units = (W.seq_start + 32 * (int64_t)W.b) * bp.f.H * bp.ds_pitch32;
    const int nqb = (n + 31) >> 5;
    return bp.ds + row_units * 64 + (int64_t)W.h * nqb * bp.ds_pitch32 * 2048;
}

typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
constexpr int kKeyBlock = 128, kQueryTile = 64;  // geometry of the key-stationary kernel

// The tiles of 64 query rows that the key-stationary kernel visits for the 128 keys starting at S0: rows at or after
// the first key (all rows if a contextual prefix sees every key), up to the last row whose window still reaches the
// block (targets sit at id max_id); inside that range a tile without a valid pair is passed over.
struct KeyBlockWalk {
    int first, end;
    bool scan;
    __device__ __forceinline__ void init(const SeqMask& M, bool has_targets, int S0, int n) {
        const int S1 = (S0 + kKeyBlock < n ? S0 + kKeyBlock : n) - 1;
        int q_hi = n - 1;
        if (M.w > 0 && M.f == 0) {
            const int id1 = M.id(S1);
            const bool targets_reach = has_targets && M.max_id - id1 <= M.w;
            if (!targets_reach) {
                const int hi = id1 + M.w + M.shift;
                q_hi = hi < q_hi ? hi : q_hi;
            }
        }
        end = q_hi / kQueryTile + 1;
        first = M.c > 0 ? 0 : S0 / kQueryTile;
        scan = M.w > 0 || M.c > 0 || has_targets;
    }
    __device__ __forceinline__ bool visits(const SeqMask& M, int jt, int S0, int n) const {
        if (jt < first || jt >= end) return false;
        if (!scan) return true;
        const int r1 = (jt + 1) * kQueryTile < n ? (jt + 1) * kQueryTile - 1 : n - 1;
        return M.classify(jt * kQueryTile, r1, S0, kKeyBlock) != 0;
    }
    __device__ __forceinline__ int next(const SeqMask& M, int jt, int S0, int n) const {
        jt = jt < first ? first : jt;
        while (jt < end && !visits(M, jt, S0, n)) ++jt;
        return jt < end ? jt : end;
    }
};

// Class of the block of 32 query rows from r0 against the 32 keys from s0 (both inside the sequence or past its end):
// 0 nothing valid, 1 masked, 2 all valid.  The key-stationary kernel stores dS for a block iff the class is not 0 and
// its walk visits the tile of the block.  `plain` (causal only: no window, contextual prefix or targets) takes a
// shortcut with the same answers.
__device__ __forceinline__ int block_class32(const SeqMask& M, bool plain, int r0, int s0, int n) {
    if (r0 >= n || s0 >= n) return 0;
    if (plain) {
        if (r0 + 31 < s0) return 0;
        return (r0 > s0 + 31 && r0 + 31 < n && s0 + 31 < n) ? 2 : 1;
    }
    const int r1 = r0 + 31 < n ? r0 + 31 : n - 1;
    int cls = M.classify(r0, r1, s0, 32);
    if (cls == 2 && r0 + 31 >= n) cls = 1;
    return cls;
}

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

// The same in two pieces whose instructions stay where they are written (the compiler does not look into the asm, so
// the wait state between a transcendental instruction and the first ordinary one that reads its result is spelled out
// where no other instruction stands between them).
__device__ __forceinline__ float sigma_pinned(float t) {
    float s;
    asm volatile("v_exp_f32 %0, %1\n\ts_nop 0\n\tv_add_f32 %0, 1.0, %0\n\tv_rcp_f32 %0, %0" : "=v"(s) : "v"(t));
    return s;
}
// p = t * sigma;  dS = dp * (sigma + p * (ln2 * sigma - ln2)).  WAIT: nothing was issued since sigma_pinned.
template <bool WAIT>
__device__ __forceinline__ void silu_and_slope_pinned(float t, float dp, float sig, float& p, float& ds) {
    const float ln2 = 0.6931471805599453f;
    if (WAIT) asm volatile("s_nop 0");
    asm volatile("v_mul_f32 %0, %2, %3\n\tv_fma_f32 %1, %5, %3, -%5\n\tv_fma_f32 %1, %0, %1, %3\n\tv_mul_f32 %1, %4, %1"
                 : "=&v"(p), "=&v"(ds)
                 : "v"(t), "v"(sig), "v"(dp), "s"(ln2));
}

// ---- key-stationary kernel: dK, dV ---------------------------------------------------------------------------------

// Per-lane constants of the mask predicate for one key.  In row POSITIONS the rows that see a key are a union of
// intervals and a point (ids are non-decreasing in the position): [rlo, rhi] from "id(key) + 1 <= id(row) <= id(key) + w",
// [r2lo, n) for the rows whose window min_full_attn_seq_len lifts, [0, crows) for the contextual rows, and the key's own
// row.
struct KeyMask {
    int pos, ids;
    int rlo, rhi, r2lo, crows;
    __device__ __forceinline__ void init(const SeqMask& M, int key_pos) {
        constexpr int kNone = 1 << 30;
        pos = key_pos;
        ids = M.id(key_pos);
        const bool clamped = M.idclamp != 0x7fffffff;  // targets given: ids stop at max_id
        rlo = (clamped && ids + 1 > M.max_id) ? kNone : ids + 1 + M.shift;
        const int w = M.w < kNone ? M.w : kNone;
        rhi = (M.w == 0 || (clamped && ids + w >= M.max_id)) ? kNone : ids + w + M.shift;
        r2lo = kNone;
        if (M.w > 0 && M.f > 0) {
            const int first_full = M.max_id - M.f;
            const int r2 = first_full <= 0 ? 0 : first_full + M.shift;
            r2lo = r2 > rlo ? r2 : rlo;
        }
        crows = (M.c > 0 && ids < M.max_id) ? M.shift + 1 : 0;
    }
    // rows at or past the end of the sequence are padding of the last tile
    __device__ __forceinline__ bool valid(const SeqMask& M, int row_pos) const {
        const int idr = M.id(row_pos);
        const int wr = (M.w == 0 || (M.f > 0 && idr >= M.max_id - M.f)) ? 0x7fffffff : M.w;
        const bool ok = (row_pos == pos) | ((unsigned)(idr - ids - 1) < (unsigned)wr) | ((M.c > 0) & (idr == 0) & (ids < M.max_id));
        return ok & (row_pos < M.n);
    }
    // Bit d = the row at position p0 + d sees this key, d = 0 .. 31 (the same predicate from the intervals).
    __device__ __forceinline__ unsigned valid_bits(int p0, int n) const {
        auto upto = [](int b) -> unsigned {  // bits 0 .. b (none if b < 0, all if b >= 31)
            const int bb = b > 31 ? 31 : (b < 0 ? 0 : b);
            return b < 0 ? 0u : 0xFFFFFFFFu >> (31 - bb);
        };
        auto from = [](int a) -> unsigned {  // bits a .. 31 (all if a <= 0, none if a > 31)
            const int aa = a < 0 ? 0 : (a > 31 ? 31 : a);
            return a > 31 ? 0u : 0xFFFFFFFFu << aa;
        };
        const int self = pos - p0;
        const unsigned own = (unsigned)self < 32u ? 1u << (self & 31) : 0u;
        const unsigned m = (from(rlo - p0) & upto(rhi - p0)) | from(r2lo - p0) | upto(crows - 1 - p0) | own;
        return m & upto(n - 1 - p0);
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

// The key-stationary kernel has two 128-row accumulators and K, V in registers: one wave per SIMD, and on this
// hardware a wave's own VALU work does not run while its MFMAs do, so what counts is the length of the one instruction
// stream.  It is software-pipelined over blocks of 32 query rows with three blocks in flight: every step issues the
// S and dP products of block i + 1, the pointwise work (sigmoid, slope, rounding) on block i, and the dV and dK
// products of block i - 1, slot by slot (two MFMAs, their LDS operand requests, one accumulator element), with the
// copies of the tile after next spread over the slots.  Tiles of 64 query rows sit in three LDS slots; the one barrier
// per tile comes when nobody can still read the tile before, whose slot the next copy overwrites.
template <class TT, int DQK, int DV, int NW, int BN, bool STORE>
__global__ __launch_bounds__(NW * 64, 1) void hstu_bwd_dkdv_kernel(const BwdParams bp) {
    typedef typename TT::vec8 vec8;
    static_assert(BN == kQueryTile && NW * 32 == kKeyBlock, "two blocks of 32 query rows per tile, four waves of 32 keys");
    const FwdParams& p = bp.f;
    constexpr int BM = NW * 32;  // key rows per workgroup
    constexpr int KS = DQK / 16, VS = DV / 16, DTK = (DQK + 31) / 32, DTV = (DV + 31) / 32;
    constexpr int QROW = DQK * 2, OROW = DV * 2;
    constexpr int QTILE = BN * QROW, OTILE = BN * OROW, STAGE = QTILE + OTILE;
    constexpr int NT = NW * 64;
    constexpr int PD = 2;  // LDS operands in flight ahead of the MFMA that uses them
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
    const int S0 = W.R0;             // first key row of the workgroup
    const int wS0 = S0 + wave * 32;  // first key row of the wave; the wave has no keys if wS0 >= n

    KeyBlockWalk walk;
    walk.init(M, p.targets != nullptr, S0, n);
    const int jt_end = walk.end;
    auto next_tile = [&](int jt) { return walk.next(M, jt, S0, n); };

    const char* qbase = p.q + (W.seq_start * p.q_rs + (int64_t)W.h * p.q_hs) * 2;
    const char* obase = bp.dout + (W.seq_start * bp.do_rs + (int64_t)W.h * bp.do_hs) * 2;
    const int64_t q_rsb = p.q_rs * 2, o_rsb = bp.do_rs * 2;
    // per-lane byte offsets of this wave's copies inside a tile that lies wholly inside the sequence (32 bits: usable
    // when 64 rows stay below 2 GB, else every tile takes the general path)
    const bool fast_copy = q_rsb < (1 << 24) && o_rsb < (1 << 24);
    constexpr int QCP = (BN * (QROW / 16) / 64 + NW - 1) / NW, OCP = (BN * (OROW / 16) / 64 + NW - 1) / NW;
    unsigned qoff[QCP], ooff[OCP];
#pragma unroll
    for (int i = 0; i < QCP; ++i) {
        const int pos = (wave + i * NW) * 64 + lane, row = pos / (QROW / 16);
        qoff[i] = (unsigned)(row * (int)q_rsb + (((pos % (QROW / 16)) ^ swz_u<QROW / 16>(row)) * 16));
    }
#pragma unroll
    for (int i = 0; i < OCP; ++i) {
        const int pos = (wave + i * NW) * 64 + lane, row = pos / (OROW / 16);
        ooff[i] = (unsigned)(row * (int)o_rsb + (((pos % (OROW / 16)) ^ swz_u<OROW / 16>(row)) * 16));
    }
    auto copy_tile = [&](int jt, int slot) {
        if (fast_copy && (jt + 1) * BN <= n) {
            const char* qb = qbase + (int64_t)jt * BN * q_rsb;
            const char* ob = obase + (int64_t)jt * BN * o_rsb;
#pragma unroll
            for (int i = 0; i < QCP; ++i)
                if (wave + i * NW < BN * (QROW / 16) / 64) global_load_lds16_soff(qb, qoff[i], smem + slot * STAGE + (wave + i * NW) * 1024);
#pragma unroll
            for (int i = 0; i < OCP; ++i)
                if (wave + i * NW < BN * (OROW / 16) / 64) global_load_lds16_soff(ob, ooff[i], smem + slot * STAGE + QTILE + (wave + i * NW) * 1024);
            return;
        }
        load_tile_u<BN, QROW, NT>(qbase, q_rsb, jt * BN, n - 1, smem + slot * STAGE, wave, lane);
        load_tile_u<BN, OROW, NT>(obase, o_rsb, jt * BN, n - 1, smem + slot * STAGE + QTILE, wave, lane);
    };

    int t_cur = next_tile(0);
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
    auto block_class = [&](int r0) { return block_class32(M, !walk.scan, r0, wS0, n); };

    // stored-dS mode: this lane's slot in the blocks of the wave's 32 keys (block row 0 of the pair)
    char* dsw = nullptr;
    if constexpr (STORE) dsw = ds_pair_base(bp, W, n) + (int64_t)(wS0 >> 5) * 2048 + (2 * l32 + g) * 16;
    const int64_t ds_qb_stride = (int64_t)bp.ds_pitch32 * 2048;

    // One step of the pipeline, in 16 slots (one per accumulator element of a block).  Three blocks of 32 query rows are
    // in flight: A -- the S and dP products of the block whose Q / dOut rows start at qn / on, into (s_n, dp_n);
    // PW -- P and dS of the block held in (s_c, dp_c), packed into (pb_o, dsb_o) WITHOUT the mask; B -- dV^T += dOut^T P
    // and dK^T += Q^T dS of the block before, whose rows start at qb / ob and whose packed P, dS are (pb_i, dsb_i).
    // The matrix pipe runs A and B while the VALU does PW; LDS operands are requested PD MFMAs ahead in each stream.
    // There is one instruction stream for all kinds of blocks (variants chosen at run time would meet again with the
    // accumulators in different registers, and the copies cost more than the work saved): a block without a valid pair
    // for the wave's keys, or past the end of the sequence, runs on whatever rows are there, and `apply_mask` below then
    // clears what must not count.
    auto step = [&](const char* qn, const char* on, f32x16_t& s_n, f32x16_t& dp_n, const f32x16_t& s_c, const f32x16_t& dp_c,
                    vec8 (&pb_o)[2], vec8 (&dsb_o)[2], const char* qb, const char* ob, const vec8 (&pb_i)[2], const vec8 (&dsb_i)[2],
                    int r0_b, bool store_b, bool do_copy, const char* cq, const char* co, char* cl) __attribute__((always_inline)) {
        constexpr int NA = OpsA::N, NB = OpsB::N, NCP = QCP + OCP;
        auto load_a = [&](int k) __attribute__((always_inline)) -> vec8 {
            return OpsA::first(k) ? *HSTU_LDS(const vec8, qn + qrow[OpsA::index(k)]) : *HSTU_LDS(const vec8, on + orow[OpsA::index(k)]);
        };
        auto load_b = [&](int k) __attribute__((always_inline)) -> vec8 {
            const int i = OpsB::index(k);
            if (OpsB::first(k)) {
                const char* b = ob + (i / DTV) * 16 * OROW;
                return read_vt_operand<TT>(b + otr[0][i % DTV], b + otr[1][i % DTV]);
            }
            const char* b = qb + (i / DTK) * 16 * QROW;
            return read_vt_operand<TT>(b + qtr[0][i % DTK], b + qtr[1][i % DTK]);
        };
        vec8 fa[PD], fb[PD];
#pragma unroll
        for (int r = 0; r < 16; ++r) s_n[r] = dp_n[r] = 0.f;
#pragma unroll
        for (int k = 0; k < PD && k < NA; ++k) fa[k] = load_a(k);
#pragma unroll
        for (int k = 0; k < PD && k < NB; ++k) fb[k] = load_b(k);
        // Slot e: one product of stream A, the first half of the pointwise work on element e (sigma), one product of
        // stream B with the copies and stores, the second half (p, the slope, dS, rounding).  A wave's VALU
        // instructions run in the shadow of its own MFMA only when few of them follow each MFMA (up to six measured:
        // 45 cycles per MFMA with six behind each one, 62 with twelve behind each pair), so the pointwise work is cut
        // into pieces of four and pinned between the products.
        auto mat_a = [&](int e) __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < NA; ++k) {
                if (k * 16 / NA != e) continue;
                if (OpsA::first(k)) s_n = TT::mfma(fa[k % PD], kreg[OpsA::index(k)], s_n);
                else dp_n = TT::mfma(fa[k % PD], vreg[OpsA::index(k)], dp_n);
                if (k + PD < NA) fa[k % PD] = load_a(k + PD);
            }
        };
        auto mat_b = [&](int e) __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < NB; ++k) {
                if (k * 16 / NB != e) continue;
                const int i = OpsB::index(k);
                if (OpsB::first(k)) dvacc[i % DTV][0] = TT::mfma(fb[k % PD], pb_i[i / DTV], dvacc[i % DTV][0]);
                else dkacc[i % DTK][0] = TT::mfma(fb[k % PD], dsb_i[i / DTK], dkacc[i % DTK][0]);
                if (k + PD < NB) fb[k % PD] = load_b(k + PD);
            }
            // the copies of a tile that lies wholly inside the sequence go out one at a time between the products
#pragma unroll
            for (int c = 0; c < NCP; ++c) {
                if (c * 16 / NCP != e) continue;
                if (do_copy) {
                    if (c < QCP) {
                        if (wave + c * NW < BN * (QROW / 16) / 64) global_load_lds16_soff(cq, qoff[c], cl + (wave + c * NW) * 1024);
                    } else {
                        if (wave + (c - QCP) * NW < BN * (OROW / 16) / 64)
                            global_load_lds16_soff(co, ooff[c - QCP], cl + QTILE + (wave + (c - QCP) * NW) * 1024);
                    }
                }
            }
            if constexpr (STORE) if (store_b) {
                char* dst = dsw + (r0_b >> 5) * ds_qb_stride;
                if (e == 0) *(vec8*)dst = dsb_i[0];
                if (e == 2) *(vec8*)(dst + 1024 + (((2 * l32 + g) * 16) ^ 128) - (2 * l32 + g) * 16) = dsb_i[1];
            }
        };
        float sg, pe[2], de[2];
        unsigned pk[4], dk[4];
        auto pw_a = [&](int e) __attribute__((always_inline)) { sg = sigma_pinned(s_c[e]); };
        auto pw_b = [&](int e) __attribute__((always_inline)) {
            silu_and_slope_pinned<(NB < 16)>(s_c[e], dp_c[e], sg, pe[e & 1], de[e & 1]);
            if (e & 1) {
                pk[(e >> 1) & 3] = TT::pack2_pinned(pe[0], pe[1]);
                dk[(e >> 1) & 3] = TT::pack2_pinned(de[0], de[1]);
            }
            if (e == 7 || e == 15) {
                pb_o[e >> 3] = __builtin_bit_cast(vec8, (u32x4_t){pk[0], pk[1], pk[2], pk[3]});
                dsb_o[e >> 3] = __builtin_bit_cast(vec8, (u32x4_t){dk[0], dk[1], dk[2], dk[3]});
            }
        };
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            __builtin_amdgcn_sched_barrier(0);
            mat_a(e);
            __builtin_amdgcn_sched_barrier(0);
            pw_a(e);
            __builtin_amdgcn_sched_barrier(0);
            mat_b(e);
            __builtin_amdgcn_sched_barrier(0);
            pw_b(e);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // Clear the entries of a packed block (first query row r0) that the mask removes: everything for class 0, the
    // pairs the predicate rejects for class 1.  Works on the rounded values, so whatever the pointwise step made of
    // rows that do not exist (even a NaN) goes away.
    auto apply_mask = [&](int cls, int r0, vec8 (&pb_o)[2], vec8 (&dsb_o)[2]) __attribute__((always_inline)) {
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
            pb_o[h] = __builtin_bit_cast(vec8, __builtin_bit_cast(u32x4_t, pb_o[h]) & m);
            dsb_o[h] = __builtin_bit_cast(vec8, __builtin_bit_cast(u32x4_t, dsb_o[h]) & m);
        }
    };

    if (t_cur < jt_end) {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the first tiles have landed
        __syncthreads();
        f32x16_t sx, dpx, sy, dpy;  // block 0 of a tile lives in x, block 1 in y
        vec8 pbx[2], dsbx[2], pby[2], dsby[2];
#pragma unroll
        for (int r = 0; r < 16; ++r) sy[r] = dpy[r] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) pby[0][j] = pby[1][j] = dsby[0][j] = dsby[1][j] = 0;
        int slot = 0;
        int clsx = block_class(t_cur * BN);
        // products of the first block; the other two stages run on zeros
        step(smem, smem + QTILE, sx, dpx, sy, dpy, pbx, dsbx, smem, smem + QTILE, pby, dsby, 0, false, false, nullptr, nullptr, nullptr);
        // Stores count in vmcnt like the tile copies, in order: the wait for a copy may leave the stores issued after
        // it outstanding (two per block whose dV / dK products ran since).
        int stores_x = 0;
        int clsy_prev = 0, r0_prev = 0;
        const char* qt_prev = smem;
        while (true) {
            const char* qt = smem + slot * STAGE;
            const char* ot = qt + QTILE;
            // block 1 of this tile: products; block 0: pointwise work; block 1 of the tile before: dV, dK
            const int clsy = block_class(t_cur * BN + 32);
            step(qt + 32 * QROW, ot + 32 * OROW, sy, dpy, sx, dpx, pbx, dsbx, qt_prev + 32 * QROW, qt_prev + QTILE + 32 * OROW, pby, dsby,
                 r0_prev, clsy_prev != 0, false, nullptr, nullptr, nullptr);
            apply_mask(clsx, t_cur * BN, pbx, dsbx);
            const bool more = t_nxt < jt_end;
            int t_nn = jt_end, cslot = 0;
            bool inline_copy = false;
            const char* qn = qt;  // after the last tile the products of the "next" block run on this one and are dropped
            if (more) {
                // the next tile, copied during the last one, has landed
                const int younger = STORE ? stores_x + (clsy_prev != 0 ? 2 : 0) : 0;
                if (younger == 4) __builtin_amdgcn_s_waitcnt(0x0F74);
                else if (younger == 2) __builtin_amdgcn_s_waitcnt(0x0F72);
                else __builtin_amdgcn_s_waitcnt(0x0F70);
                __syncthreads();  // ... for every wave; and nobody reads the tile before this one any more
                t_nn = next_tile(t_nxt + 1);
                const int nslot = slot == 2 ? 0 : slot + 1;
                cslot = nslot == 2 ? 0 : nslot + 1;
                inline_copy = fast_copy && t_nn < jt_end && (t_nn + 1) * BN <= n;
                // a tile that reaches past the end of the sequence (the last one) is copied here, with its rows clamped
                if (t_nn < jt_end && !inline_copy) copy_tile(t_nn, cslot);
                // stores issued after the last copy and before the next wait for it
                stores_x = inline_copy ? 0 : (clsx != 0 ? 2 : 0);
                qn = smem + nslot * STAGE;
            }
            // block 0 of the next tile: products; block 1 of this tile: pointwise work; block 0 of this tile: dV, dK
            step(qn, qn + QTILE, sx, dpx, sy, dpy, pby, dsby, qt, ot, pbx, dsbx, t_cur * BN, clsx != 0, inline_copy,
                 qbase + (int64_t)t_nn * BN * q_rsb, obase + (int64_t)t_nn * BN * o_rsb, smem + cslot * STAGE);
            apply_mask(clsy, t_cur * BN + 32, pby, dsby);
            clsy_prev = clsy;
            r0_prev = t_cur * BN + 32;
            qt_prev = qt;
            if (!more) break;
            clsx = block_class(t_nxt * BN);
            t_cur = t_nxt;
            t_nxt = t_nn;
            slot = slot == 2 ? 0 : slot + 1;
        }
        // dV, dK of the very last block (the other two stages run on what is there and are dropped)
        step(qt_prev, qt_prev + QTILE, sy, dpy, sx, dpx, pbx, dsbx, qt_prev + 32 * QROW, qt_prev + QTILE + 32 * OROW, pby, dsby,
             r0_prev, clsy_prev != 0, false, nullptr, nullptr, nullptr);
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
            // one instruction stream for every kind of block (see the key-stationary kernel): a block without a valid
            // pair runs like the others and its dS is cleared afterwards
            const int cls = M.classify(wR0, wR1, s0, 32);
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
                    d8[j] = dp[r] * gr;
                }
                dsb[half] = TT::pack8(d8);
            }
            if (cls != 2) {
                typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
                const unsigned keys = cls == 1 ? row.valid_bits(s0 + 4 * g) : 0u;  // bit d: key s0 + 4 g + d is visible
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    u32x4_t m;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const int r = 8 * half + 2 * w, d = 8 * (r >> 2) + (r & 3);  // elements r, r + 1: keys d, d + 1
                        const unsigned lo = (unsigned)__builtin_amdgcn_sbfe((int)keys, d, 1);
                        const unsigned hi = (unsigned)__builtin_amdgcn_sbfe((int)keys, d + 1, 1);
                        m[w] = (lo & 0xFFFFu) | (hi & 0xFFFF0000u);
                    }
                    dsb[half] = __builtin_bit_cast(vec8, __builtin_bit_cast(u32x4_t, dsb[half]) & m);
                }
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

// ---- dQ from stored dS --------------------------------------------------------------------------------------------

// dQ^T[d, q] += K^T dS^T with dS read back from the blocks the key-stationary kernel stored: one product instead of
// three and no pointwise work; the kernel streams 2 bytes per (query, key) pair from HBM and is bound by that.
// A workgroup owns NW * 32 query rows and walks the key tiles as the forward kernel does.  K tiles are shared through
// LDS (three slots, one barrier per tile); each wave copies the two blocks of ITS 32 rows per tile straight into a
// private LDS ring (three slots as well, so two tiles -- 2 x NW x 4 KB -- are in flight per workgroup) and reads them
// with transposing reads: the stored image has the key in the lane and four consecutive query rows per 8 bytes, the
// B operand wants the query row in the lane and consecutive keys.  A block is used iff the key-stationary kernel
// stored it (same walk, same classification).
template <class TT, int DQK, int NW, int BN>
__global__ __launch_bounds__(NW * 64, 1) void hstu_bwd_dq_stored_kernel(const BwdParams bp) {
    typedef typename TT::vec8 vec8;
    static_assert(BN == 64 && TT::ES == 2, "two blocks of 32 keys per tile, 16-bit operands");
    const FwdParams& p = bp.f;
    constexpr int BM = NW * 32;
    constexpr int DTK = (DQK + 31) / 32;
    constexpr int KROW = DQK * 2, KTILE = BN * KROW, KCH = KROW / 16;
    constexpr int KINSTR = BN * KCH / 64, KPW = (KINSTR + NW - 1) / NW;  // K copies per tile, per wave
    constexpr int NSLOT = 3, DSBYTES = 4096;                            // per wave and slot: two blocks
    constexpr int PER_STEP = KPW + 4;
    static_assert(PER_STEP <= 15, "wait immediates below");
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    char* const ds_lds = smem + NSLOT * KTILE;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, l32 = lane & 31;

    Work W;
    if (!bwd_decode<BM>(p, W, blockIdx.x, false)) return;
    const SeqMask& M = W.M;
    const int n = W.n;
    kv_tile_range(M, W.u, W.R0, W.R1, BN, W.jt_begin, W.jt_end);
    const int jt_end = W.jt_end;
    const int wq0 = W.m0 + wave * 32;  // the wave has no rows if wq0 >= n

    const char* kbase = p.k + (W.seq_start * p.k_rs + (int64_t)W.h * p.k_hs) * 2;
    const int64_t k_rsb = p.k_rs * 2;
    // the wave's row of blocks; a wave without rows copies the last row of blocks and uses nothing of it
    const int nqb = (n + 31) >> 5;
    const int qb = (wq0 >> 5) < nqb ? (wq0 >> 5) : nqb - 1;
    const char* dsrow = ds_pair_base(bp, W, n) + (int64_t)qb * bp.ds_pitch32 * 2048;
    char* const my_ds = ds_lds + wave * (NSLOT * DSBYTES);

    auto copy_step = [&](int jt, int slot) {
        // every wave issues KPW copies of the K tile (the last ones may repeat a neighbour's: same bytes, same place)
#pragma unroll
        for (int i = 0; i < KPW; ++i) {
            int inst = wave + i * NW;
            inst = inst < KINSTR ? inst : KINSTR - 1;
            const int pos = inst * 64 + lane;
            const int row = pos / KCH;
            const int logical = (pos % KCH) ^ swz_u<KCH>(row);
            int grow = jt * BN + row;
            grow = grow > n - 1 ? n - 1 : grow;
            global_load_lds16(kbase + (int64_t)grow * k_rsb + logical * 16, smem + slot * KTILE + inst * 1024);
        }
        const char* src = dsrow + (int64_t)(2 * jt) * 2048 + lane * 16;
#pragma unroll
        for (int i = 0; i < 4; ++i) global_load_lds16_nt(src + i * 1024, my_ds + slot * DSBYTES + i * 1024);
    };

    int ktr[2][DTK], krow_unused[DQK / 16];
    lds_offsets_u<DQK>(krow_unused, ktr, lane);
    // transposing reads of a stored block: lane (g, half, jrow, q4) supplies key 16 tt + 8 sec + 4 g + jrow, query rows
    // 16 half + 4 q4 .. + 3, which sit in the 16 bytes of source lane (key, q4 & 1) of half `half`, upper 8 if q4 >= 2
    int dtr[2][2];
    {
        const int i16 = lane & 15, half = (lane >> 4) & 1, jrow = i16 >> 2, q4 = i16 & 3;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int sec = 0; sec < 2; ++sec) {
                const int key = 16 * tt + 8 * sec + 4 * g + jrow;
                dtr[tt][sec] = (64 * half + ((2 * key + (q4 & 1)) ^ (8 * half))) * 16 + (q4 >> 1) * 8;
            }
    }

    f32x16_t dqacc[DTK][1];
#pragma unroll
    for (int dt = 0; dt < DTK; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dqacc[dt][0][r] = 0.f;

    int t_cur = next_valid_tile<BN>(W, W.jt_begin);
    int t_nxt = t_cur < jt_end ? next_valid_tile<BN>(W, t_cur + 1) : jt_end;
    if (t_cur < jt_end) copy_step(t_cur, 0);
    if (t_nxt < jt_end) copy_step(t_nxt, 1);
    int slot = 0;
    const bool has_targets = p.targets != nullptr;
    while (t_cur < jt_end) {
        // this tile has landed; the next one (if any) may still be in flight
        if (t_nxt < jt_end) __builtin_amdgcn_s_waitcnt(0x0F70 | PER_STEP);
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();  // K of this tile is there for every wave, and nobody reads the tile before it any more
        const int t_nn = t_nxt < jt_end ? next_valid_tile<BN>(W, t_nxt + 1) : jt_end;
        if (t_nn < jt_end) copy_step(t_nn, slot == 0 ? 2 : slot - 1);
        const char* kt = smem + slot * KTILE;
        const char* dt_lds = my_ds + slot * DSBYTES;
        const int S0 = (t_cur * BN) & ~(kKeyBlock - 1);
        KeyBlockWalk walk;
        walk.init(M, has_targets, S0, n);
        const bool visited = wq0 < n && walk.visits(M, wq0 / kQueryTile, S0, n);
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            const int s0 = t_cur * BN + sub * 32;
            if (!visited || block_class32(M, !walk.scan, wq0, s0, n) == 0) continue;
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const vec8 dsT = read_vt_operand<TT>(dt_lds + sub * 2048 + dtr[tt][0], dt_lds + sub * 2048 + dtr[tt][1]);
                const char* kb = kt + (sub * 32 + tt * 16) * KROW;
#pragma unroll
                for (int dt = 0; dt < DTK; ++dt)
                    dqacc[dt][0] = TT::mfma(read_vt_operand<TT>(kb + ktr[0][dt], kb + ktr[1][dt]), dsT, dqacc[dt][0]);
            }
        }
        t_cur = t_nxt;
        t_nxt = t_nn;
        slot = slot == 2 ? 0 : slot + 1;
    }
    store_output<TT, DTK>(dqacc, 0, bp.dq, W.seq_start, wq0 + l32, n, bp.dq_rs, bp.dq_hs, W.h, g, bp.gscale, DQK);
}


}  // namespace hstu
