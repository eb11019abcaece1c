// HSTU jagged attention forward for gfx950 (CDNA4): device code.
//
// One workgroup owns BM = NW*QT*32 consecutive query rows of one (sequence, head) pair and walks
// the key/value rows of that sequence in tiles of BN.  All matrix work is on
// v_mfma_f32_32x32x16_{bf16,f16}, computed transposed so that no register shuffle is needed
// between the two products:
//
//   S^T[kv, q] = K[kv, :] . Q[q, :]^T        A = K tile (LDS),   B = Q (registers, loaded once)
//   P^T        = silu-part(S^T), masked      in registers, packed to 16 bit
//   O^T[dv, q] += V^T[dv, kv] . P^T[kv, q]   A = V tile (LDS, transposing read), B = P^T (registers)
//
// The accumulator layout of a 32x32 MFMA holds, per lane, one column (a query row) and sixteen
// rows (kv positions); taken eight at a time those sixteen values are exactly the B operand of
// the second product, provided the A operand (V^T) enumerates the kv rows in the same order,
// which the ds_read_b64_tr_b16 addressing below arranges.
//
// silu(alpha*s)/N is evaluated as  s * rcp(1 + exp2(-alpha*log2(e)*s))  per element and the
// common factor alpha/N is applied once to the fp32 output.  There is no row max / row sum:
// HSTU attention is pointwise (pt_hstu_attention.py:151-182 of the reference).
//
// K and V tiles go HBM -> LDS with global_load_lds_dwordx4 (no register staging), double
// buffered.  An XOR swizzle of the 16-byte chunk index with the row index keeps both the
// b128 reads of K and the transposing reads of V off each other's banks; it is applied on the
// global side of the copy because the LDS side of a direct load is fixed (lane i -> base + 16 i).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hstu {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(2))) int i32x2_t;

#define HSTU_LDS(T, p) ((__attribute__((address_space(3))) T*)(p))
#define HSTU_GLB(T, p) ((const __attribute__((address_space(1))) T*)(p))

struct FwdParams {
    const char* q;
    const char* k;
    const char* v;
    char* o;
    int64_t q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, o_rs, o_hs;  // strides in elements
    const void* offsets;
    const void* targets;
    int offsets_i64, targets_i64;
    int B, H;
    int num_mb;         // row blocks per (sequence, head) pair in the grid
    int max_seq_len;
    int delta;          // 0 = full attention
    int w, c, f;        // max_attn_len, contextual_seq_len, min_full_attn_seq_len
    float c1;           // -alpha * log2(e)
    float oscale;       // alpha / max_seq_len
};

struct Bf16 {
    typedef bf16x8_t vec8;
    typedef __bf16 elem;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
struct Fp16 {
    typedef f16x8_t vec8;
    typedef _Float16 elem;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// Per-sequence mask state; every field is wave-uniform.
struct SeqMask {
    int n;        // sequence length
    int shift;    // contextual_seq_len - 1 (0 if none): position -> id is max(pos - shift, 0)
    int idclamp;  // ids are clamped to this (max_id when targets are given, else INT_MAX)
    int max_id;   // id of the first target (or one past the last id)
    int w, c, f;
    __device__ __forceinline__ int id(int pos) const {
        int x = pos - shift;
        x = x < 0 ? 0 : x;
        return x > idclamp ? idclamp : x;
    }
    // Classify rows [r_lo, r_hi] (inclusive, all < n) against kv positions [s_lo, s_lo + bn):
    // 0 = no valid pair, 1 = some, 2 = every pair valid and no padding column.
    __device__ __forceinline__ int classify(int r_lo, int r_hi, int s_lo, int bn) const {
        if (s_lo >= n || r_hi < r_lo) return 0;
        int s_hi = s_lo + bn - 1;
        bool padded = s_hi >= n;
        if (padded) s_hi = n - 1;
        int idr_lo = id(r_lo), idr_hi = id(r_hi), ids_lo = id(s_lo), ids_hi = id(s_hi);
        if (!padded && ids_hi < idr_lo && (w == 0 || idr_hi - ids_lo <= w)) return 2;
        bool diag = s_lo <= r_hi && r_lo <= s_hi;
        bool caus = ids_lo < idr_hi && (w == 0 || f > 0 || idr_lo - ids_hi <= w);
        bool ctx = c > 0 && idr_lo == 0 && ids_lo < max_id;
        return (diag || caus || ctx) ? 1 : 0;
    }
};

// Chunk swizzles.  LDS has 64 banks of 4 bytes (256 bytes per clock); a row of CH 16-byte chunks is
// stored with chunk index XOR f(row).
//
// K tile, read with ds_read_b128 by 16 lanes at a time (16 consecutive rows, same logical chunk): f must
// send those 16 rows to 16 different 16-byte slots of the 256-byte bank line.
template <int CH>
__device__ __forceinline__ int swz_k(int row) {
    static_assert(CH == 4 || CH == 8 || CH == 16, "row of 64, 128 or 256 bytes");
    return (row / (16 / CH)) & (CH - 1);
}
// V tile, read with ds_read_b64_tr_b16: one instruction touches 8 rows (4 per half-wave) x one 64-byte
// segment, 8 bytes per lane.  f must send rows r..r+3 to four different 64-byte bank groups and rows
// r, r+4 to different 32-byte halves of a group.
template <int CH>
__device__ __forceinline__ int swz_v(int row) {
    static_assert(CH == 4 || CH == 8 || CH == 16, "row of 64, 128 or 256 bytes");
    const int half_swap = ((row >> 2) & 1) << 1;
    if (CH == 16) return ((row & 3) << 2) | half_swap;
    if (CH == 8) return (((row >> 1) & 1) << 2) | half_swap;
    return half_swap;
}

// 16 bytes per lane, global memory -> LDS at lds_base + 16*lane (lds_base is wave-uniform and goes
// through M0).  Written as inline assembly on purpose: the compiler then does not know that an LDS
// write is in flight and does not put a vmcnt(0) wait in front of the next LDS read, which would
// expose the whole HBM latency of the prefetch.  The kernel waits for these copies itself
// (s_waitcnt vmcnt(0) followed by the workgroup barrier) before the tile is read.  The s_nop covers the
// one wait state the hardware wants between a scalar write of M0 and an LDS-DMA instruction; the
// compiler's hazard pass does not look inside an asm block.
__device__ __forceinline__ void global_load_lds16(const char* src, const char* lds_base) {
    const unsigned m0 = (unsigned)(uintptr_t)HSTU_LDS(const char, lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0), "v"(src) : "memory");
}

// Copy `ROWS` rows of `ROWBYTES` bytes from global memory into LDS with the chunk swizzle.
// Rows at or beyond `n_rows_valid` re-read the last valid row (their products are masked).
template <int ROWS, int ROWBYTES, int NTHREADS, bool IS_V>
__device__ __forceinline__ void load_tile_to_lds(const char* gbase, int64_t row_stride_bytes, int row0,
                                                 int last_row, char* lds_tile, int wave, int lane) {
    constexpr int CH = ROWBYTES / 16;                // 16-byte chunks per row
    constexpr int INSTR = ROWS * CH / 64;            // wave-wide copies per tile
    constexpr int NWAVES = NTHREADS / 64;
    static_assert(INSTR % NWAVES == 0, "tile copy must split evenly over the waves");
#pragma unroll
    for (int i = 0; i < INSTR / NWAVES; ++i) {
        int inst = wave + i * NWAVES;
        int p = inst * 64 + lane;
        int row = p / CH;
        int phys = p % CH;
        int logical = phys ^ (IS_V ? swz_v<CH>(row) : swz_k<CH>(row));
        int grow = row0 + row;
        grow = grow > last_row ? last_row : grow;
        const char* src = gbase + (int64_t)grow * row_stride_bytes + logical * 16;
        global_load_lds16(src, lds_tile + inst * 1024);
    }
}

// One kv tile for one wave: S^T = K Q^T, P^T = s*sigmoid(alpha s) (masked if MASKED), O^T += V^T P^T.
// `sp0` is the sequence position of this lane's first kv slot: tile start + 4*(lane/32).
template <class TT, int DQK, int DV, int QT, int BN, bool MASKED>
__device__ __forceinline__ void tile_compute(const char* kt, const char* vt, const typename TT::vec8 (&qreg)[QT][DQK / 16],
                                             f32x16_t (&oacc)[DV / 32][QT], const int (&kaddr)[DQK / 16],
                                             const int (&vaddr)[2][DV / 32], float c1, const SeqMask& M, int sp0,
                                             const int (&row_pos)[QT], const int (&row_lo)[QT], const int (&row_w)[QT],
                                             const bool (&row_ctx)[QT]) {
    typedef typename TT::vec8 vec8;
    typedef typename TT::elem elem;
    constexpr int NS = BN / 32, KS = DQK / 16, DT = DV / 32, KROW = DQK * 2, VROW = DV * 2;
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
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float x = s[sub][qt][r];
                float e = __builtin_amdgcn_exp2f(x * c1);
                float pr = x * __builtin_amdgcn_rcpf(1.0f + e);
                if (MASKED) {
                    int sp = sp0 + sub * 32 + 8 * (r >> 2) + (r & 3);
                    int ids = M.id(sp);
                    bool ok = (sp == row_pos[qt]) | ((unsigned)(ids - row_lo[qt]) < (unsigned)row_w[qt]) |
                              (row_ctx[qt] & (ids < M.max_id));
                    pr = ok ? pr : 0.f;
                }
                pb[sub][qt][r >> 3][r & 7] = (elem)pr;
            }
    // ---- O^T += V^T P^T
#pragma unroll
    for (int sub = 0; sub < NS; ++sub)
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const char* vb = vt + (sub * 32 + tt * 16) * VROW;
                s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(HSTU_LDS(s16x4_t, vb + vaddr[0][dt]));
                s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(HSTU_LDS(s16x4_t, vb + vaddr[1][dt]));
                s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                vec8 a = __builtin_bit_cast(vec8, both);
#pragma unroll
                for (int qt = 0; qt < QT; ++qt) oacc[dt][qt] = TT::mfma(a, pb[sub][qt][tt], oacc[dt][qt]);
            }
}

template <class TT, int DQK, int DV, int QT, int NW, int BN, int OCC>
__global__ __launch_bounds__(NW * 64, OCC) void hstu_fwd_kernel(const FwdParams p) {
    typedef typename TT::vec8 vec8;
    typedef typename TT::elem elem;
    constexpr int BM = NW * QT * 32;
    constexpr int NS = BN / 32;
    constexpr int KS = DQK / 16;
    constexpr int DT = DV / 32;
    constexpr int KROW = DQK * 2, VROW = DV * 2;
    constexpr int KCH = DQK / 8, VCH = DV / 8;
    constexpr int KTILE = BN * KROW, VTILE = BN * VROW, STAGE = KTILE + VTILE;
    constexpr int NT = NW * 64;
    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5;      // which half of the k-slots of an MFMA operand this lane holds
    const int l32 = lane & 31;    // operand row (A) / column (B, C) this lane holds

    // ---- which (row block, sequence, head): workgroup ids go round-robin over the 8 XCDs, so ids
    // congruent mod 8 share an L2.  All row blocks of one (sequence, head) pair stay on one XCD,
    // heaviest (last) row block first.
    const int bid = blockIdx.x;
    const int xcd = bid & 7;
    const int slot = bid >> 3;
    const int pair = (slot / p.num_mb) * 8 + xcd;
    if (pair >= p.B * p.H) return;
    const int mb = p.num_mb - 1 - (slot % p.num_mb);
    const int b = pair / p.H;
    const int h = pair - b * p.H;

    int64_t seq_start, seq_end;
    if (p.offsets_i64) {
        seq_start = ((const int64_t*)p.offsets)[b];
        seq_end = ((const int64_t*)p.offsets)[b + 1];
    } else {
        seq_start = ((const int*)p.offsets)[b];
        seq_end = ((const int*)p.offsets)[b + 1];
    }
    int n = (int)(seq_end - seq_start);
    n = n > p.max_seq_len ? p.max_seq_len : n;      // rows past max_seq_len do not exist for the reference either
    const int nq = p.delta > 0 ? p.delta : n;
    const int m0 = mb * BM;
    const int rbase = p.delta > 0 ? n - p.delta : 0;  // sequence position of query row 0
    if (n <= 0 || m0 >= nq || rbase < 0) return;

    int t = 0;
    if (p.targets) t = p.targets_i64 ? (int)((const int64_t*)p.targets)[b] : ((const int*)p.targets)[b];
    SeqMask M;
    M.n = n;
    M.w = p.w;
    M.c = p.c;
    M.f = p.f;
    M.shift = p.c > 0 ? p.c - 1 : 0;
    const int u = n - t;
    M.max_id = u - M.shift;
    M.idclamp = p.targets ? M.max_id : 0x7fffffff;

    // rows of this workgroup / this wave, as sequence positions (inclusive ranges)
    const int m1 = (m0 + BM < nq ? m0 + BM : nq);
    const int R0 = rbase + m0, R1 = rbase + m1 - 1;
    const int wq0 = m0 + wave * (QT * 32);
    const int wR0 = rbase + wq0;
    const int wR1 = (wq0 + QT * 32 < nq ? rbase + wq0 + QT * 32 : rbase + nq) - 1;  // < wR0 if the wave has no rows

    // kv range of the workgroup
    const int idr_lo = M.id(R0);
    const bool ctx_rows = p.c > 0 && idr_lo == 0;
    int kv_hi = R1 + 1;
    if (ctx_rows && u > kv_hi) kv_hi = u;
    if (kv_hi > n) kv_hi = n;
    int kv_lo = 0;
    if (p.w > 0 && p.f == 0 && !ctx_rows && idr_lo - p.w > 0) kv_lo = idr_lo - p.w + M.shift;
    const int jt_end = (kv_hi + BN - 1) / BN;
    int jt = kv_lo / BN;
    while (jt < jt_end && M.classify(R0, R1, jt * BN, BN) == 0) ++jt;

    const char* kbase = p.k + (seq_start * p.k_rs + (int64_t)h * p.k_hs) * 2;
    const char* vbase = p.v + (seq_start * p.v_rs + (int64_t)h * p.v_hs) * 2;
    const int64_t k_rsb = p.k_rs * 2, v_rsb = p.v_rs * 2;

    if (jt < jt_end) {
        load_tile_to_lds<BN, KROW, NT, false>(kbase, k_rsb, jt * BN, n - 1, smem, wave, lane);
        load_tile_to_lds<BN, VROW, NT, true>(vbase, v_rsb, jt * BN, n - 1, smem + KTILE, wave, lane);
    }

    // ---- Q operand (B of the first product): lane holds Q[row l32][16 ks + 8 g .. +8)
    vec8 qreg[QT][KS];
    {
        const int64_t qrow0 = p.delta > 0 ? (int64_t)b * p.delta : seq_start;
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            int ql = wq0 + qt * 32 + l32;
            ql = ql < nq ? ql : nq - 1;
            const char* qp = p.q + ((qrow0 + ql) * p.q_rs + (int64_t)h * p.q_hs) * 2 + g * 16;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) qreg[qt][ks] = *(const vec8*)(qp + ks * 32);
        }
    }

    // ---- per-lane mask constants for the rows this lane owns
    int row_pos[QT], row_lo[QT], row_w[QT];
    bool row_ctx[QT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        int rp = wR0 + qt * 32 + l32;
        int idr = M.id(rp);
        int wr = (p.w == 0 || (p.f > 0 && idr >= M.max_id - p.f)) ? 0x7fffffff : p.w;
        row_pos[qt] = rp;
        row_w[qt] = wr;
        row_lo[qt] = idr - wr;
        row_ctx[qt] = p.c > 0 && idr == 0;
    }

    // ---- LDS read addresses (byte offsets inside a K / V tile), constant over the kv loop
    // K, A operand: row sub*32 + l32, logical chunk 2 ks + g
    int kaddr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = l32 * KROW + (((2 * ks + g) ^ swz_k<KCH>(l32)) * 16);
    // V^T, A operand via ds_read_b64_tr_b16.  Within each group of 16 lanes, lane 4j+q supplies the
    // address of 4 consecutive dv of kv row j; the hardware hands lane i the four kv rows of dv i.
    // Operand lane l must end up with dv = l32 and kv slots {4g+0..3} (first read), {8+4g+0..3} (second).
    int vaddr[2][DT];
    {
        const int i16 = lane & 15, half = (lane >> 4) & 1;
        const int jrow = i16 >> 2, q4 = i16 & 3;
#pragma unroll
        for (int sec = 0; sec < 2; ++sec) {
            int row = 8 * sec + 4 * g + jrow;  // + 32 sub + 16 t
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                int chunk = dt * 4 + 2 * half + (q4 >> 1);
                vaddr[sec][dt] = row * VROW + ((chunk ^ swz_v<VCH>(row)) * 16) + (q4 & 1) * 8;
            }
        }
    }

    f32x16_t oacc[DT][QT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][qt][r] = 0.f;

    int stage = 0;
    while (jt < jt_end) {
        int jn = jt + 1;
        while (jn < jt_end && M.classify(R0, R1, jn * BN, BN) == 0) ++jn;

        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this tile's direct-to-LDS copies have landed
        __syncthreads();                      // ... for every wave, and the other stage is no longer read
        if (jn < jt_end) {
            char* nxt = smem + (stage ^ 1) * STAGE;
            load_tile_to_lds<BN, KROW, NT, false>(kbase, k_rsb, jn * BN, n - 1, nxt, wave, lane);
            load_tile_to_lds<BN, VROW, NT, true>(vbase, v_rsb, jn * BN, n - 1, nxt + KTILE, wave, lane);
        }

        const int cls = M.classify(wR0, wR1, jt * BN, BN);
        const char* kt = smem + stage * STAGE;
        if (cls == 2) {
            tile_compute<TT, DQK, DV, QT, BN, false>(kt, kt + KTILE, qreg, oacc, kaddr, vaddr, p.c1, M, jt * BN + 4 * g,
                                                     row_pos, row_lo, row_w, row_ctx);
        } else if (cls == 1) {
            tile_compute<TT, DQK, DV, QT, BN, true>(kt, kt + KTILE, qreg, oacc, kaddr, vaddr, p.c1, M, jt * BN + 4 * g,
                                                    row_pos, row_lo, row_w, row_ctx);
        }
        jt = jn;
        stage ^= 1;
    }

    // ---- epilogue: out[q, dv] = alpha/N * O^T[dv, q]; lane holds 4 consecutive dv per (dt, r/4)
    {
        const int64_t orow0 = p.delta > 0 ? (int64_t)b * p.delta : seq_start;
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            int ql = wq0 + qt * 32 + l32;
            if (ql < nq) {
                char* op = p.o + ((orow0 + ql) * p.o_rs + (int64_t)h * p.o_hs) * 2 + g * 8;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        typedef __attribute__((ext_vector_type(4))) elem elem4;
                        elem4 o4;
#pragma unroll
                        for (int i = 0; i < 4; ++i) o4[i] = (elem)(oacc[dt][qt][r4 * 4 + i] * p.oscale);
                        *(elem4*)(op + (dt * 32 + r4 * 8) * 2) = o4;
                    }
            }
        }
    }
}

}  // namespace hstu
