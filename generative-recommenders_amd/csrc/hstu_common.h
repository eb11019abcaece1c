// HSTU jagged attention forward for gfx950 (CDNA4): device code.
//
// One workgroup owns BM = NW*QT*32 consecutive query rows of one (sequence, head) pair and walks
// the key/value rows of that sequence in tiles of BN.  All matrix work is on
// v_mfma_f32_32x32x16_{bf16,f16,fp8_fp8}, computed transposed so that no register shuffle is needed
// between the two products:
//
//   S^T[kv, q] = K[kv, :] . Q[q, :]^T        A = K tile (LDS),   B = Q (registers, loaded once)
//   P^T        = silu-part(S^T), masked      in registers, packed to the operand type
//   O^T[dv, q] += V^T[dv, kv] . P^T[kv, q]   A = V tile (LDS, transposing read), B = P^T (registers)
//
// The accumulator layout of a 32x32 MFMA holds, per lane, one column (a query row) and sixteen
// rows (kv positions); taken eight at a time those sixteen values are exactly the B operand of
// the second product, provided the A operand (V^T) enumerates the kv rows in the same order,
// which the ds_read_b64_tr_b16 / ds_read_b64_tr_b8 addressing below arranges.
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
#define HSTU_CONST(T, p) ((const __attribute__((address_space(4))) T*)(p))

__device__ __forceinline__ int64_t uniform64(int64_t x) {
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(uint64_t)x);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)((uint64_t)x >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// What decode_work needs of FwdParams, gathered (by the host: fill_decode_params in the API source) into one block of
// 32 dwords that a wave fetches with two wide scalar loads and one wait.  Read field by field from FwdParams, every
// field is fetched where it is first needed, behind whatever branch that is, with a wait of its own -- some forty
// dependent round trips to the scalar cache per decoded item.
struct DecodeParams {
    const int* items;
    const int* nitems;
    const int* order;
    const void* offsets;
    const void* targets;
    int items_cap, kv_splits, kv_chunk, c, pairs_per_xcd, num_mb, B, H;
    int uniform, max_seq_len, offsets_i64, targets_i64, delta, w, f, pad0;
    unsigned mb_magic, mb_shift, h_magic, h_shift;
    int pad1[2];
};
static_assert(sizeof(DecodeParams) == 128, "two loads of 16 dwords");

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
    const int* order;   // NULL, or sequence indices sorted by decreasing length (scheduling only)
    int num_mb;         // row blocks per (sequence, head) pair in the grid
    int pairs_per_xcd;  // ceil(B*H / 8)
    int slots_per_xcd;  // work items per XCD = pairs_per_xcd * num_mb * kv_splits
    int* queue;         // NULL, or 8 counters 64 bytes apart (one per XCD) handing out work items
    // NULL, or the work lists built by hstu_plan_kernel: record i of list xcd (8 ints at items[(xcd * items_cap + i) * 8])
    // = {b, h, row block, n, seq_start (low, high), targets, 0}: everything decode_work would otherwise have to look up
    // through two dependent loads.  Heaviest class first, nitems[xcd] entries.  Without them item i of an XCD is decoded
    // arithmetically and may turn out to hold no work (a row block past the end of a short sequence).
    const int* items;
    const int* nitems;
    int items_cap;
    int max_seq_len;
    int uniform;        // 1: every sequence is exactly max_seq_len long (total_kv == B * max_seq_len under the caller's contract):
                        // sequence b starts at row b * max_seq_len, and nobody reads the offsets
    unsigned mb_magic, mb_shift, h_magic, h_shift;  // division by num_mb and by H without a divider (see fast_div)
    int delta;          // 0 = full attention
    int w, c, f;        // max_attn_len, contextual_seq_len, min_full_attn_seq_len
    float c1;           // -alpha * log2(e): Q is multiplied by it when loaded
    float oscale;       // (alpha / max_seq_len) / c1 = -1 / (max_seq_len * log2(e)); 0 if alpha == 0
    // attn_scale of the reference (pt_hstu_attention.py:152-165): a factor per query row, or one for all, that takes the
    // place of 1 / max_seq_len.  NULL = none; `oscale_unit` is `oscale` without the 1 / max_seq_len.
    const float* attn_scale;
    int attn_scale_per_row;
    float oscale_unit;
    // Split of the kv range of a row block into runs of `kv_chunk` tiles, each taken by its own workgroup; the
    // grid holds `kv_splits` workgroups per row block (1 = off) and those past the end of a short range exit at
    // once.  Each run writes its unscaled fp32 accumulators to partial[split][row][head][dv] (dense) and run 0
    // writes the number of runs to split_counts[(b * H + h) * num_mb + row block]; a second kernel adds the
    // runs in a fixed order.
    int kv_splits;
    int kv_chunk;
    float* partial;
    int64_t partial_stride;  // floats per split = total_q * H * dv
    int* split_counts;
    alignas(64) DecodeParams dec;  // copies of the fields above that decode_work reads
};

// Element types.  ES = bytes per element; `vec8` = eight elements = one MFMA operand of a lane;
// `out_elem` = type of the output tensor; PRESCALE_Q: multiply Q by c1 when it is loaded (otherwise c1 is
// applied to the accumulator); `silu` maps one accumulator value to the P value that is rounded and
// packed by `pack8`, leaving a constant factor to the output scale.
// %4 .. %7 <- t / (1 + 2^t) for the four values a .. d, side by side; operands %4 .. %7 of the enclosing asm are scratch
// registers, and the two packed results go to p and q
#define HSTU_SILU4(a, b, c, d, p, q)                                                                                   \
    "v_exp_f32 %4, " a "\n\tv_exp_f32 %5, " b "\n\tv_exp_f32 %6, " c "\n\tv_exp_f32 %7, " d "\n\t"                     \
    "v_add_f32 %4, 1.0, %4\n\tv_add_f32 %5, 1.0, %5\n\tv_add_f32 %6, 1.0, %6\n\tv_add_f32 %7, 1.0, %7\n\t"             \
    "v_rcp_f32 %4, %4\n\tv_rcp_f32 %5, %5\n\tv_rcp_f32 %6, %6\n\tv_rcp_f32 %7, %7\n\t"                                 \
    "v_mul_f32 %4, " a ", %4\n\tv_mul_f32 %5, " b ", %5\n\tv_mul_f32 %6, " c ", %6\n\tv_mul_f32 %7, " d ", %7\n\t"     \
    "v_cvt_pk_bf16_f32 " p ", %4, %5\n\tv_cvt_pk_bf16_f32 " q ", %6, %7\n\t"
struct Bf16 {
    static constexpr bool PAIRWISE = false;
    typedef bf16x8_t vec8;
    typedef __bf16 elem;
    typedef __bf16 out_elem;
    static constexpr int ES = 2;
    static constexpr bool PRESCALE_Q = true;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // accumulator already holds t = c1*s; p = t * sigmoid(alpha s) = t / (1 + 2^t)
    static __device__ __forceinline__ float silu(float t, float) {
        return t * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
    }
    static __device__ __forceinline__ vec8 pack8(const float (&p)[8]) {
        vec8 r;
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = (elem)p[j];
        return r;
    }
    // two values rounded as pack8 rounds them, by an instruction that stays where it is written
    static __device__ __forceinline__ unsigned pack2_pinned(float a, float b) {
        unsigned r;
        asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
        return r;
    }
    // silu + pack8 of eight accumulator values as ONE fixed instruction sequence: four chains side by side, so that no
    // instruction waits for the one in front of it (a transcendental result is not there for the very next
    // instruction), in four scratch registers.  Left to the compiler the same work comes out four wide in some copies
    // of the loop body and strictly serial -- one scratch register, a wait state behind every exp and rcp -- in others,
    // depending on what else is live around it.
    static constexpr bool PINNED_SILU = true;
    static __device__ __forceinline__ vec8 silu_pack8_pinned(const float (&t)[8]) {
        unsigned p0, p1, p2, p3;
        float e0, e1, e2, e3;
        asm volatile(HSTU_SILU4("%8", "%9", "%10", "%11", "%0", "%1") HSTU_SILU4("%12", "%13", "%14", "%15", "%2", "%3")
                     : "=&v"(p0), "=&v"(p1), "=&v"(p2), "=&v"(p3), "=&v"(e0), "=&v"(e1), "=&v"(e2), "=&v"(e3)
                     : "v"(t[0]), "v"(t[1]), "v"(t[2]), "v"(t[3]), "v"(t[4]), "v"(t[5]), "v"(t[6]), "v"(t[7]));
        typedef __attribute__((ext_vector_type(4))) unsigned u4;
        const u4 r = {p0, p1, p2, p3};
        return __builtin_bit_cast(vec8, r);
    }
};
// The second instruction of a pair writes the other half of the register the first one wrote, and reads that register
// to do so; four independent instructions in between cover the latency of the first (the compiler does not see into
// the asm, so nothing else would).  Operands 0-3: results, 4-7: packed fp16 pairs.
#define HSTU_F16_PAIRS(op)                                                                                              \
    "v_" op "_f16_e32 %0, %4\n\tv_" op "_f16_e32 %1, %5\n\tv_" op "_f16_e32 %2, %6\n\tv_" op "_f16_e32 %3, %7\n\t"      \
    "v_" op "_f16_sdwa %0, %4 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"                            \
    "v_" op "_f16_sdwa %1, %5 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"                            \
    "v_" op "_f16_sdwa %2, %6 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"                            \
    "v_" op "_f16_sdwa %3, %7 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1"
typedef __attribute__((ext_vector_type(2))) _Float16 h2_t;
// r[j] = 1 / (1 + 2^t[j]) for four packed pairs: the transcendental instructions take one value each, the additions
// two.  2^t beyond fp16 is inf and gives 0.
__device__ __forceinline__ void sigmoid_f16_pairs(const h2_t (&t)[4], h2_t (&r)[4]) {
    h2_t e[4];
    asm(HSTU_F16_PAIRS("exp") : "=&v"(e[0]), "=&v"(e[1]), "=&v"(e[2]), "=&v"(e[3]) : "v"(t[0]), "v"(t[1]), "v"(t[2]), "v"(t[3]));
#pragma unroll
    for (int j = 0; j < 4; ++j) e[j] = e[j] + (h2_t){(_Float16)1.0f, (_Float16)1.0f};
    asm(HSTU_F16_PAIRS("rcp") : "=&v"(r[0]), "=&v"(r[1]), "=&v"(r[2]), "=&v"(r[3]) : "v"(e[0]), "v"(e[1]), "v"(e[2]), "v"(e[3]));
}
#undef HSTU_F16_PAIRS

struct Fp16 {
    static constexpr bool PAIRWISE = false;
    static constexpr bool PINNED_SILU = false;
    typedef f16x8_t vec8;
    typedef _Float16 elem;
    typedef _Float16 out_elem;
    static constexpr int ES = 2;
    static constexpr bool PRESCALE_Q = true;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float silu(float t, float) {
        return t * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
    }
    static __device__ __forceinline__ vec8 pack8(const float (&p)[8]) {
        vec8 r;
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = (elem)p[j];
        return r;
    }
    static __device__ __forceinline__ unsigned pack2_pinned(float a, float b) {
        unsigned r, t;
        asm volatile("v_cvt_f16_f32 %0, %2\n\tv_cvt_f16_f32 %1, %3\n\tv_pack_b32_f16 %0, %0, %1" : "=&v"(r), "=&v"(t) : "v"(a), "v"(b));
        return r;
    }
};
// fp16 operands (rounded copies of fp32 inputs), fp32 output straight from the accumulators.
struct Fp16F32 : Fp16 {
    typedef float out_elem;
};
// OCP e4m3 (torch.float8_e4m3fn) inputs with per-tensor scales, bf16 output.  Both products run on
// v_mfma_f32_32x32x16_fp8_fp8.  Q cannot be pre-scaled in 8 bits, so c1 (which here also carries
// q_scale*k_scale) multiplies the accumulator.  P is kept in e4m3 as 16 * t * sigmoid: the factor 16 puts
// typical magnitudes (|t| around 1e-2) into the normal range of e4m3 (2^-6 .. 448); p is unbounded only
// towards -inf (t -> -inf), where it is clamped to the largest finite e4m3 value.
struct Fp8 {
    typedef long vec8;
    typedef unsigned char elem;
    typedef __bf16 out_elem;
    static constexpr int ES = 1;
    static constexpr bool PRESCALE_Q = false;
    static constexpr bool PINNED_SILU = false;
    static constexpr float PSCALE = 16.0f;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a, b, c, 0, 0, 0);
    }
    // Four of these operands side by side are one operand of v_mfma_f32_32x32x64_f8f6f4, which runs at twice the
    // rate of the 16-deep instruction (the only 8-bit rate that reaches the part's fp8 peak).  Which 32 of the 64
    // k positions a lane group supplies does not matter as long as A and B agree, so the 8-byte pieces that the
    // 16-deep scheme loads are simply used four at a time.
    static __device__ __forceinline__ f32x16_t mfma64(const vec8 (&a)[4], const vec8 (&b)[4], f32x16_t c) {
        typedef __attribute__((ext_vector_type(4))) long l4;
        typedef __attribute__((ext_vector_type(8))) int i8;
        const l4 av = {a[0], a[1], a[2], a[3]}, bv = {b[0], b[1], b[2], b[3]};
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(__builtin_bit_cast(i8, av), __builtin_bit_cast(i8, bv), c, 0, 0, 0, 0, 0,
                                                               0);
    }
    static __device__ __forceinline__ float silu(float raw, float c1) {
        const float t = raw * c1;
        const float e = __builtin_amdgcn_exp2f(t);
        const float d = __builtin_fmaf(e, 1.0f / PSCALE, 1.0f / PSCALE);  // (1 + 2^t) / 16
        const float p = t * __builtin_amdgcn_rcpf(d);
        return __builtin_fmaxf(p, -448.0f);
    }
    static __device__ __forceinline__ vec8 pack8(const float (&p)[8]) {
        int lo = 0, hi = 0;
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(p[0], p[1], lo, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(p[2], p[3], lo, true);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(p[4], p[5], hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(p[6], p[7], hi, true);
        return (long)(((unsigned long)(unsigned)hi << 32) | (unsigned)lo);
    }
    // Eight scores of a tile without mask, two at a time in packed fp16 (P is kept to three mantissa bits, so fp16's
    // eleven are plenty): t = raw * c1 in fp32, then per pair one conversion, two exp2, one packed add, two rcp, one
    // packed multiply and one conversion to two e4m3 values that also applies the factor 16 and saturates -- 29 VALU
    // issue cycles per score instead of 34.  The conversions run with MODE.FP16_OVFL = 1 (saturate at +-448 instead of
    // NaN), everything in front of them with 0, so that a 2^t beyond fp16 is inf and p = t * 0 = 0 as it should be.
    static constexpr bool PAIRWISE = true;
    static __device__ __forceinline__ vec8 silu_pack8(const float (&raw)[8], float c1) {
        // stage by stage over the four pairs, so that no instruction waits for the one in front of it
        h2_t t[4], r[4], p[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] = __builtin_bit_cast(h2_t, __builtin_amdgcn_cvt_pkrtz(raw[2 * j] * c1, raw[2 * j + 1] * c1));
        sigmoid_f16_pairs(t, r);
#pragma unroll
        for (int j = 0; j < 4; ++j) p[j] = t[j] * r[j];
        // (volatile, and the mode switch inside: the compiler does not know that the conversions depend on the mode)
        unsigned lo, hi;
        asm volatile(
            "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1\n\ts_nop 1\n\t"
            "v_cvt_scalef32_pk_fp8_f16 %0, %2, %6\n\tv_cvt_scalef32_pk_fp8_f16 %1, %4, %6\n\t"
            "v_cvt_scalef32_pk_fp8_f16 %0, %3, %6 op_sel:[0,0,1]\n\tv_cvt_scalef32_pk_fp8_f16 %1, %5, %6 op_sel:[0,0,1]\n\t"
            "s_nop 0\n\ts_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 0"
            : "=&v"(lo), "=&v"(hi)
            : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(1.0f / PSCALE));
        return (long)(((unsigned long)hi << 32) | lo);
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
    static_assert(CH == 2 || CH == 4 || CH == 8 || CH == 16, "row of 32 .. 256 bytes");
    return (row / (16 / CH)) & (CH - 1);
}
// V tile of 16-bit elements, read with ds_read_b64_tr_b16: one instruction touches 8 rows (4 per
// half-wave) x one 64-byte segment, 8 bytes per lane.  f must send rows r..r+3 to four different 64-byte
// bank groups and rows r, r+4 to different 32-byte halves of a group.
// V tile of 8-bit elements (128-byte rows), read with ds_read_b64_tr_b8: a half-wave touches rows
// {0..3, 8..11} + 4g, 32 bytes each (two 16-byte chunks 2dt, 2dt+1); rows of equal parity share a
// 128-byte half of the bank line, so f spreads rows {0,2,8,10} (and {1,3,9,11}) over chunk pairs.
template <int CH, int ES>
__device__ __forceinline__ int swz_v(int row) {
    static_assert(CH == 2 || CH == 4 || CH == 8 || CH == 16, "row of 32 .. 256 bytes");
    if (ES == 1) {
        if (CH == 8) return (((row >> 1) & 1) | (((row >> 3) & 1) << 1)) << 1;
        return 0;
    }
    if (CH == 2) return 0;  // 32-byte rows (dv = 16): two chunks, nothing to spread
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

// The same copy for data that is read once: marked non-temporal so that it does not displace what the other copies
// of the kernel keep re-reading from L2.
__device__ __forceinline__ void global_load_lds16_nt(const char* src, const char* lds_base) {
    const unsigned m0 = (unsigned)(uintptr_t)HSTU_LDS(const char, lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" : : "s"(m0), "v"(src) : "memory");
}

// What one workgroup has to do; every field is wave-uniform.
struct Work {
    int b, h;
    int64_t seq_start;
    int n;            // sequence length (clipped to max_seq_len)
    int nq;           // query rows of this sequence (n, or delta_size)
    int m0;           // first query row of the workgroup (index into the nq rows)
    int m1;           // one past its last query row
    int rbase;        // sequence position of query row 0 (n - delta_size in delta mode)
    int u;            // number of non-target positions
    int split;        // which run of the kv range this workgroup takes (0 when the range is not split)
    int nsplit;       // number of non-empty runs of this row block
    int block_id;     // (b * H + h) * num_mb + row block
    int R0, R1;       // sequence positions of the workgroup's first and last row (inclusive)
    int jt_begin;     // first kv tile that can hold a valid pair
    int jt_end;       // one past the last such tile
    bool skip_scan;   // true if tiles inside [jt_begin, jt_end) may hold no valid pair (window / targets / contextual)
    SeqMask M;
};

// Tiles [jt_begin, jt_end) of `bn` kv rows that can hold a valid pair for rows R0..R1 (sequence positions) of a
// sequence with `u` non-target positions.
__device__ __forceinline__ void kv_tile_range(const SeqMask& M, int u, int R0, int R1, int bn, int& jt_begin, int& jt_end) {
    const int idr_lo = M.id(R0);
    const bool ctx_rows = M.c > 0 && idr_lo == 0;
    int kv_hi = R1 + 1;
    if (ctx_rows && u > kv_hi) kv_hi = u;
    if (kv_hi > M.n) kv_hi = M.n;
    int kv_lo = 0;
    if (M.w > 0 && M.f == 0 && !ctx_rows && idr_lo - M.w > 0) kv_lo = idr_lo - M.w + M.shift;
    jt_end = (kv_hi + bn - 1) / bn;
    jt_begin = kv_lo / bn;
}

// Query rows [m0, m1) of row block `mb` (of `bm` rows) of a sequence with `nq` query rows; false if there is no such
// block.  In the full form without a kv split the blocks are aligned to the END of the sequence, so that the partly
// filled block is the first one -- the one with the fewest keys -- instead of the last one, which has the most: a block
// costs its kv range however many of its rows exist, and a batch of short ragged sequences otherwise spends
// bm / (2 n) of its steps on rows that do not exist (a quarter of them at n = 2 bm).  Otherwise (delta form, kv
// split: there the row-block index is also the key of the partial sums) they start at row 0.
__device__ __forceinline__ bool row_block_rows(int nq, int mb, int bm, bool end_aligned, int& m0, int& m1) {
    if (end_aligned) {
        const int m = (nq + bm - 1) / bm;
        if (mb >= m) return false;
        m1 = nq - (m - 1 - mb) * bm;
        m0 = m1 - bm > 0 ? m1 - bm : 0;
        return true;
    }
    m0 = mb * bm;
    m1 = m0 + bm < nq ? m0 + bm : nq;
    return m0 < nq;
}
__device__ __forceinline__ bool row_blocks_end_aligned(const FwdParams& p) { return p.delta == 0 && p.kv_splits <= 1; }

// The pair (sequence in rank order, head) that is number `i` of XCD `xcd`: the pairs are dealt to the XCDs back and
// forth (0 .. 7, 7 .. 0, ...).  With the sequences ranked by length a plain round-robin gives XCD 0 the longest pair of
// every eight and XCD 7 the shortest, several per cent more work on the one than on the other.
__device__ __forceinline__ int pair_of(int i, int xcd) { return i * 8 + ((i & 1) ? 7 - xcd : xcd); }

// x / d for 0 <= x < 2^31 with constants the host derives from d (fast_div_constants in the API source): with
// l = ceil(log2 d) and m = floor(2^(31+l) / d) + 1, x / d = (x * m) >> (31 + l); magic 0 stands for d = 1.
__device__ __forceinline__ int fast_div(int x, unsigned magic, unsigned shift) {
    return magic ? (int)(__umulhi((unsigned)x, magic) >> shift) : x;
}

// Decode work item `bid` (the workgroup id in a one-item-per-workgroup launch) of the launch whose FwdParams are the
// kernel's first argument.  Workgroup ids go round-robin
// over the 8 XCDs, so ids congruent mod 8 share an L2: all row blocks of one (sequence, head) pair stay on one
// XCD, heaviest block first.  Returns false if the item holds no work.
template <int BM, int BN>
__device__ __forceinline__ bool decode_work(Work& w, int bid) {
    // the block of parameters, straight from the kernel argument segment: FwdParams is the kernels' first argument
    typedef __attribute__((ext_vector_type(16))) int i32x16_t;
    struct Two { i32x16_t a, b; };
    const __attribute__((address_space(4))) char* kernarg = (const __attribute__((address_space(4))) char*)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(kernarg));  // fetched again for every item, not kept in registers across the item loop
    const __attribute__((address_space(4))) i32x16_t* block = (const __attribute__((address_space(4))) i32x16_t*)(kernarg + __builtin_offsetof(FwdParams, dec));
    const Two raw = {block[0], block[1]};
    const DecodeParams p = __builtin_bit_cast(DecodeParams, raw);
    const int xcd = bid & 7;
    int slot = bid >> 3;
    // the splits of one row block are neighbours on one XCD
    w.split = 0;
    if (p.kv_splits > 1) {
        const int s0 = slot / p.kv_splits;
        w.split = slot - s0 * p.kv_splits;
        slot = s0;
    }
    // Heaviest work first.  Within a pair that is the last row block -- except that with a contextual prefix
    // the first row block (its contextual rows see every non-target key) is the heaviest of all and runs
    // many times longer than the others, so the first row blocks of all pairs are launched before anything else.
    int pair_local, mb;
    int64_t seq_start, seq_end;
    int t = 0;
    if (p.items) {
        // everything straight from the list: one load
        if (slot >= HSTU_CONST(int, p.nitems)[xcd]) return false;
        typedef __attribute__((ext_vector_type(8))) int i32x8_t;
        const i32x8_t rec = HSTU_CONST(i32x8_t, p.items)[(int64_t)xcd * p.items_cap + slot];
        w.b = __builtin_amdgcn_readfirstlane(rec[0]);
        w.h = __builtin_amdgcn_readfirstlane(rec[1]);
        mb = __builtin_amdgcn_readfirstlane(rec[2]);
        seq_start = (int64_t)(((uint64_t)(unsigned)rec[5] << 32) | (unsigned)rec[4]);
        seq_end = seq_start + rec[3];
        t = rec[6];
    } else {
        if (p.c > 0) {
            if (slot < p.pairs_per_xcd) {
                pair_local = slot;
                mb = 0;
            } else {
                const int s2 = slot - p.pairs_per_xcd;
                pair_local = s2 / (p.num_mb - 1);
                mb = p.num_mb - 1 - (s2 - pair_local * (p.num_mb - 1));
            }
        } else {
            pair_local = fast_div(slot, p.mb_magic, p.mb_shift);
            mb = p.num_mb - 1 - (slot - pair_local * p.num_mb);
        }
        const int pair = pair_of(pair_local, xcd);
        if (pair >= p.B * p.H) return false;
        const int rseq = fast_div(pair, p.h_magic, p.h_shift);
        w.h = pair - rseq * p.H;
        // `order` lists the sequences longest first, so that long sequences start early and are dealt evenly
        // over the XCDs; it changes the schedule, never the result
        // The index arrays are read-only for the whole launch and their addresses are wave-uniform: reading
        // them through the constant address space makes these scalar loads (scalar cache, a fraction of the
        // latency of a vector load), which matters because they are chained at the start of every item.
        w.b = p.order ? HSTU_CONST(int, p.order)[rseq] : rseq;
        if (p.uniform) {
            seq_start = (int64_t)w.b * p.max_seq_len;
            seq_end = seq_start + p.max_seq_len;
        } else if (p.offsets_i64) {
            seq_start = HSTU_CONST(int64_t, p.offsets)[w.b];
            seq_end = HSTU_CONST(int64_t, p.offsets)[w.b + 1];
        } else {
            seq_start = HSTU_CONST(int, p.offsets)[w.b];
            seq_end = HSTU_CONST(int, p.offsets)[w.b + 1];
        }
        if (p.targets) t = p.targets_i64 ? (int)HSTU_CONST(int64_t, p.targets)[w.b] : HSTU_CONST(int, p.targets)[w.b];
    }
    // Values read from memory are the same for every lane; say so, so that everything derived from
    // them (loop bounds, tile classes, base addresses) lives in scalar registers.
    w.seq_start = uniform64(seq_start);
    int n = __builtin_amdgcn_readfirstlane((int)(seq_end - seq_start));
    n = n > p.max_seq_len ? p.max_seq_len : n;  // rows past max_seq_len do not exist for the reference either
    w.n = n;
    w.nq = p.delta > 0 ? p.delta : n;
    w.rbase = p.delta > 0 ? n - p.delta : 0;
    if (n <= 0 || w.rbase < 0 || !row_block_rows(w.nq, mb, BM, (p.delta == 0 && p.kv_splits <= 1), w.m0, w.m1)) return false;

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

    w.R0 = w.rbase + w.m0;
    w.R1 = w.rbase + w.m1 - 1;
    kv_tile_range(M, w.u, w.R0, w.R1, BN, w.jt_begin, w.jt_end);
    w.nsplit = 1;
    w.block_id = (w.b * p.H + w.h) * p.num_mb + mb;
    if (p.kv_splits > 1) {
        w.nsplit = (w.jt_end - w.jt_begin + p.kv_chunk - 1) / p.kv_chunk;
        const int b = w.jt_begin + w.split * p.kv_chunk;
        if (b >= w.jt_end) return false;  // a short range has fewer runs than the grid provides
        w.jt_end = b + p.kv_chunk < w.jt_end ? b + p.kv_chunk : w.jt_end;
        w.jt_begin = b;
    }
    w.skip_scan = p.w > 0 || p.c > 0 || p.targets != nullptr;
    return true;
}

// Inclusive prefix sum over the 64 lanes of a wave with data-parallel-primitive moves: shifts by 1, 2, 4, 8
// inside each row of 16 lanes (lanes without a source add 0), then lane 15 of rows 0 and 2 is added to rows 1
// and 3, then lane 31 to rows 2 and 3.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
    return v;
}

#define HSTU_PLAN_THREADS 1024
// Builds the work lists of the persistent kernels: one workgroup per XCD walks the (sequence, head) pairs that
// XCD owns (pair_of(i, xcd), sequences taken in `order` if given) and lists every row block that exists,
// sorted by weight class (floor(log2(kv tiles)), heaviest class first; within a class in pair order, within a
// pair heaviest block first).  Heavy-first across the whole list keeps the end of the launch made of small
// items, items of one class and pair stay neighbours (they share K/V through the L2), and row blocks past the
// end of short sequences never become items.  A stable counting sort: the candidate items in pair-major order
// are cut into 256 equal runs, one per thread; count per thread and class, scan over the threads, place.
static __global__ __launch_bounds__(HSTU_PLAN_THREADS) void hstu_plan_kernel(const FwdParams p, int bm, int bn, int* nitems, int* items) {
    constexpr int NC = 12;    // classes: up to 2^11 = 2048 tiles and more
    constexpr int NT = HSTU_PLAN_THREADS, NW = NT / 64;
    constexpr int CACHE = 32768;  // candidates whose class is remembered between the two walks
    __shared__ int cnt[NC][NT];
    __shared__ int wave_sum[NC][NW];
    __shared__ int cbase[NC];
    __shared__ signed char cls[CACHE];  // weight class of candidate k, -1 = no such row block
    const int xcd = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int c = 0; c < NC; ++c) cnt[c][tid] = 0;
    const int num_mb = p.num_mb;
    const int total = p.pairs_per_xcd * num_mb;  // candidates: every row block a pair could have
    const int run = (total + NT - 1) / NT;
    const int k_end = (tid + 1) * run < total ? (tid + 1) * run : total;
    auto walk = [&](bool place) {
        int cur_pl = -1, b = 0, h = 0, n = 0, nq = 0, rbase = 0, u = 0, t = 0;
        int64_t seq_start = 0;
        bool live = false;
        SeqMask M;
        auto put = [&](int pos, int mb) {  // record `pos` of this XCD's list
            if (pos < p.items_cap) {
                typedef __attribute__((ext_vector_type(4))) int i32x4;
                i32x4* rec = (i32x4*)(items + 8 * ((int64_t)xcd * p.items_cap + pos));
                rec[0] = (i32x4){b, h, mb, n};
                rec[1] = (i32x4){(int)(unsigned)(uint64_t)seq_start, (int)(unsigned)((uint64_t)seq_start >> 32), t, 0};
            }
        };
        for (int k = tid * run; k < k_end; ++k) {
            const int pl = k / num_mb;
            const int mb = num_mb - 1 - (k - pl * num_mb);  // heaviest block of a pair first
            if (place && k < CACHE && cls[k] < 0) continue;  // second walk: known not to exist
            if (!place && k < CACHE) cls[k] = -1;
            if (pl != cur_pl) {
                cur_pl = pl;
                const int pair = pair_of(pl, xcd);
                live = pair < p.B * p.H;
                if (live) {
                    const int rseq = pair / p.H;
                    b = p.order ? p.order[rseq] : rseq;
                    h = pair - rseq * p.H;
                    seq_start = p.offsets_i64 ? ((const int64_t*)p.offsets)[b] : (int64_t)((const int*)p.offsets)[b];
                    const int64_t len = (p.offsets_i64 ? ((const int64_t*)p.offsets)[b + 1] : (int64_t)((const int*)p.offsets)[b + 1]) - seq_start;
                    n = len > p.max_seq_len ? p.max_seq_len : (int)len;
                    nq = p.delta > 0 ? p.delta : n;
                    rbase = p.delta > 0 ? n - p.delta : 0;
                    live = n > 0 && rbase >= 0;
                    t = 0;
                    if (p.targets) t = p.targets_i64 ? (int)((const int64_t*)p.targets)[b] : ((const int*)p.targets)[b];
                    M.n = n;
                    M.w = p.w;
                    M.c = p.c;
                    M.f = p.f;
                    M.shift = p.c > 0 ? p.c - 1 : 0;
                    u = n - t;
                    M.max_id = u - M.shift;
                    M.idclamp = p.targets ? M.max_id : 0x7fffffff;
                }
            }
            int c;
            if (place && k < CACHE) {
                c = cls[k];  // the class is remembered from the first walk
            } else {
                int m0, m1;
                if (!live || !row_block_rows(nq, mb, bm, row_blocks_end_aligned(p), m0, m1)) continue;
                int jb, je;
                kv_tile_range(M, u, rbase + m0, rbase + m1 - 1, bn, jb, je);
                const int tiles = je - jb;
                if (tiles <= 0) continue;
                c = 31 - __builtin_clz((unsigned)tiles);
                c = c > NC - 1 ? NC - 1 : c;
                if (!place && k < CACHE) cls[k] = (signed char)c;
            }
            if (place) put(cbase[c] + cnt[c][tid], mb);
            cnt[c][tid] += 1;
        }
    };
    walk(false);
    __syncthreads();
    // exclusive scan over the threads for every class: within a wave by shuffles, across waves through LDS
    int excl[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int v = cnt[c][tid];
        const int incl = wave_inclusive_scan(v);
        excl[c] = incl - v;
        if (lane == 63) wave_sum[c][wave] = incl;
    }
    __syncthreads();
    if (tid < NC) {  // per class: wave sums -> exclusive prefix over the waves, and the class total
        int run_sum = 0;
        for (int w = 0; w < NW; ++w) {
            const int x = wave_sum[tid][w];
            wave_sum[tid][w] = run_sum;
            run_sum += x;
        }
        cbase[tid] = run_sum;
    }
    __syncthreads();
    if (tid == 0) {
        int start = 0;
        for (int c = NC - 1; c >= 0; --c) {  // heaviest class first
            const int x = cbase[c];
            cbase[c] = start;
            start += x;
        }
        nitems[xcd] = start < p.items_cap ? start : p.items_cap;
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) cnt[c][tid] = excl[c] + wave_sum[c][wave];
    __syncthreads();
    walk(true);
}

// First tile index >= jt that holds a valid pair for the workgroup's rows (jt_end if none).
template <int BN>
__device__ __forceinline__ int next_valid_tile(const Work& w, int jt) {
    if (w.skip_scan)
        while (jt < w.jt_end && w.M.classify(w.R0, w.R1, jt * BN, BN) == 0) ++jt;
    return jt;
}

// Per-lane constants of the mask predicate for one query row.  In key POSITIONS the predicate is a union of two
// intervals and a point: ids are non-decreasing in the position, so "id(row) - w <= id(key) <= id(row) - 1" is
// klo <= key <= khi, "contextual row and id(key) < max_id" is key < cend, and the row itself is always visible.
struct RowMask {
    int pos;    // sequence position of the row
    int lo;     // id(row) - window: key ids in [lo, lo + w) pass the causal+window test
    int w;      // window of this row (INT_MAX if unlimited)
    bool ctx;   // contextual row: sees every non-target key
    int klo, khi;  // first and last key position of the causal+window interval (khi = -1: empty)
    int cend;      // keys before this position are visible to a contextual row (0 otherwise)
    __device__ __forceinline__ void init(const SeqMask& M, int row_pos) {
        const int idr = M.id(row_pos);
        pos = row_pos;
        w = (M.w == 0 || (M.f > 0 && idr >= M.max_id - M.f)) ? 0x7fffffff : M.w;
        lo = idr - w;
        ctx = M.c > 0 && idr == 0;
        klo = lo > 0 ? lo + M.shift : 0;
        khi = idr >= 1 ? idr - 1 + M.shift : -1;
        cend = (ctx && M.max_id > 0) ? M.max_id + M.shift : 0;  // a sequence shorter than the prefix has max_id <= 0: nothing passes
    }
    __device__ __forceinline__ bool valid(const SeqMask& M, int key_pos) const {
        const int ids = M.id(key_pos);
        return (key_pos == pos) | ((unsigned)(ids - lo) < (unsigned)w) | (ctx & (ids < M.max_id));
    }
    // Bit d = the key at position p0 + d is visible, d = 0 .. 31: the same predicate from the position intervals,
    // about twenty operations for the 32 keys instead of a dozen per key.
    __device__ __forceinline__ unsigned valid_bits(int p0) const {
        auto upto = [](int b) -> unsigned {  // bits 0 .. b (none if b < 0, all if b >= 31)
            const int bb = b > 31 ? 31 : (b < 0 ? 0 : b);
            return b < 0 ? 0u : 0xFFFFFFFFu >> (31 - bb);
        };
        auto from = [](int a) -> unsigned {  // bits a .. 31 (all if a <= 0, none if a > 31)
            const int aa = a < 0 ? 0 : (a > 31 ? 31 : a);
            return a > 31 ? 0u : 0xFFFFFFFFu << aa;
        };
        const unsigned window = from(klo - p0) & upto(khi - p0);
        const unsigned prefix = upto(cend - 1 - p0);
        const int self = pos - p0;
        const unsigned own = (unsigned)self < 32u ? 1u << (self & 31) : 0u;
        return window | prefix | own;
    }
};

// P^T for one 32x32 block.  With t = c1*s, c1 = -alpha*log2(e) (for 16-bit inputs the accumulator already
// holds t because Q was pre-scaled), s*sigmoid(alpha s) = (t / c1) * rcp(1 + exp2(t)); the kernel forms
// p = t * rcp(1 + exp2(t)) (TT::silu) and leaves the constant 1/c1 to the output scale.  p is zeroed where
// the mask says so, rounded to the operand type and packed as two MFMA B operands.
// `sp0` is the sequence position of this lane's first kv slot of the block.
// MASK: 0 = every pair valid, 1 = exact general predicate, 2 = plain causal (no window, targets or
// contextual prefix: key position <= row position), which costs a compare and a select per element.
template <class TT, int MASK>
__device__ __forceinline__ void silu_pack(const f32x16_t& s, typename TT::vec8 (&pb)[2], float c1, const SeqMask& M,
                                          const RowMask& row, int sp0) {
    if constexpr (MASK == 0 && TT::PAIRWISE) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float raw[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) raw[j] = s[half * 8 + j];
            pb[half] = TT::silu_pack8(raw, c1);
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }
    if constexpr (MASK == 0 && TT::PINNED_SILU) {
        // The hardware does not interlock an MFMA result against a VALU read; the compiler counts the wait states, but
        // not for reads inside an asm block.  One read it can see (of any register of the accumulator) in front of the
        // blocks makes it count for them too.
        asm volatile("" : : "s"(__builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, (float)s[15]))));
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float t[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) t[j] = s[half * 8 + j];
            pb[half] = TT::silu_pack8_pinned(t);
        }
        return;
    }
    const int causal_room = row.pos - sp0;  // a key at offset d from sp0 is visible iff d <= causal_room
    unsigned bits = 0;
    if (MASK == 1) bits = row.valid_bits(sp0);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        // eight elements at a time, fenced, so that the scheduler cannot pile up temporaries of all sixteen
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int r = half * 8 + j;
            float pr = TT::silu(s[r], c1);
            if (MASK == 1)  // all ones or zero from the key's bit, AND-ed onto the value
                pr = __builtin_bit_cast(float, __builtin_bit_cast(int, pr) & __builtin_amdgcn_sbfe((int)bits, 8 * (r >> 2) + (r & 3), 1));
            if (MASK == 2) pr = (8 * (r >> 2) + (r & 3) <= causal_room) ? pr : 0.f;
            p[j] = pr;
        }
        pb[half] = TT::pack8(p);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// B operand of the first product for one block of 32 query rows: lane holds Q[row][16 ks + 8 g .. +8),
// multiplied by `qscale` = -alpha*log2(e) and rounded back to the 16-bit type, so that the first product
// directly yields t = -alpha*log2(e)*s, the argument of the exp2 in the sigmoid; this removes one VALU
// multiply per score element, which is what the kernel is short of.  The extra rounding of Q is of the size
// of the rounding the 16-bit inputs already carry.  Rows at or past `nq` re-read the last valid row (their
// outputs are never stored).
template <class TT, int KS>
__device__ __forceinline__ void load_q_operand(typename TT::vec8 (&qreg)[KS], const char* q, int64_t qrow0, int ql, int nq,
                                               int64_t q_rs, int64_t q_hs, int h, int g, float qscale) {
    typedef typename TT::vec8 vec8;
    constexpr int ES = TT::ES;
    ql = ql < nq ? ql : nq - 1;
    const char* qp = q + ((qrow0 + ql) * q_rs + (int64_t)h * q_hs) * ES + g * 8 * ES;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        vec8 raw = *(const vec8*)(qp + ks * 16 * ES);
        if constexpr (TT::PRESCALE_Q) {
            typedef typename TT::elem elem;
#pragma unroll
            for (int j = 0; j < 8; ++j) raw[j] = (elem)((float)raw[j] * qscale);
        }
        qreg[ks] = raw;
    }
}

// Byte offsets, inside a K tile and a V tile, of this lane's LDS reads; constant over the kv loop.
// K (A operand of the first product): row sub*32 + lane%32, logical chunk 2 ks + lane/32.
// V^T (A operand of the second product) through ds_read_b64_tr_b16: within each group of 16 lanes,
// lane 4j+q supplies the address of 4 consecutive dv of kv row j and the hardware hands lane i the four
// kv rows of dv i.  Operand lane l must end up with dv = l%32 and kv slots {4g..4g+3} (first read) and
// {8+4g..8+4g+3} (second read), g = l/32 -- the order in which the accumulator of the first product
// holds its kv rows.
template <class TT, int DQK, int DV>
__device__ __forceinline__ void lds_read_offsets(int (&kaddr)[DQK / 16], int (&vaddr)[2][(DV + 31) / 32], int lane) {
    constexpr int ES = TT::ES;
    // DV = 16 still takes one 32-row MFMA: its upper 16 dv rows read whatever follows the row in LDS and are never stored
    constexpr int KS = DQK / 16, DT = (DV + 31) / 32, KROW = DQK * ES, VROW = DV * ES, KCH = KROW / 16, VCH = VROW / 16;
    const int g = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int byte = (16 * ks + 8 * g) * ES;  // eight consecutive elements of the row
        kaddr[ks] = l32 * KROW + (((byte >> 4) ^ swz_k<KCH>(l32)) * 16) + (byte & 15);
    }
    const int i16 = lane & 15, half = (lane >> 4) & 1;
    if constexpr (ES == 2) {
        const int jrow = i16 >> 2, q4 = i16 & 3;
#pragma unroll
        for (int sec = 0; sec < 2; ++sec) {
            const int row = 8 * sec + 4 * g + jrow;  // + 32 sub + 16 t
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int chunk = dt * 4 + 2 * half + (q4 >> 1);
                vaddr[sec][dt] = row * VROW + ((chunk ^ swz_v<VCH, ES>(row)) * 16) + (q4 & 1) * 8;
            }
        }
    } else {
        // ds_read_b64_tr_b8: within 16 lanes, lanes 2j and 2j+1 supply the address of 16 consecutive dv of
        // kv row j (8 bytes each) and the hardware hands lane i the eight kv rows of dv i: one read fills
        // all eight kv slots {4g..4g+3, 8+4g..8+4g+3} of the operand.
        const int jrow = i16 >> 1, e = i16 & 1;
        const int row = 8 * (jrow >> 2) + 4 * g + (jrow & 3);  // + 32 sub + 16 t
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int chunk = dt * 2 + half;
            vaddr[0][dt] = row * VROW + ((chunk ^ swz_v<VCH, ES>(row)) * 16) + e * 8;
            vaddr[1][dt] = 0;
        }
    }
}

// A operand of the second product (32 dv x 16 kv): two transposing LDS reads of four 16-bit elements, or
// one of eight 8-bit elements.
template <class TT>
__device__ __forceinline__ typename TT::vec8 read_vt_operand(const char* lo_addr, const char* hi_addr) {
    if constexpr (TT::ES == 2) {
        s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(HSTU_LDS(s16x4_t, lo_addr));
        s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(HSTU_LDS(s16x4_t, hi_addr));
        s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(typename TT::vec8, both);
    } else {
        i32x2_t v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(HSTU_LDS(i32x2_t, lo_addr));
        return __builtin_bit_cast(typename TT::vec8, v);
    }
}

// The factor the fp32 accumulators of output row `row` (index into out, clamped by the caller) are multiplied with.
__device__ __forceinline__ float output_scale(const FwdParams& p, int64_t row) {
    if (!p.attn_scale) return p.oscale;
    return p.oscale_unit * p.attn_scale[p.attn_scale_per_row ? row : 0];
}

// out[q, dv] = oscale * O^T[dv, q] for one block of 32 query rows; the lane holds 4 consecutive dv per
// (dv tile, r/4), stored as 8 bytes.  QT is deduced from the accumulator array.
template <class TT, int DT, int QT>
__device__ __forceinline__ void store_output(const f32x16_t (&oacc)[DT][QT], int qt, char* o, int64_t orow0, int ql, int nq,
                                             int64_t o_rs, int64_t o_hs, int h, int g, float oscale,
                                             int dv_valid = 1 << 30) {
    typedef typename TT::out_elem elem;  // 16 bits, or float
    typedef __attribute__((ext_vector_type(4))) elem elem4;
    constexpr int OES = sizeof(elem);
    if (ql >= nq) return;
    char* op = o + ((orow0 + ql) * o_rs + (int64_t)h * o_hs) * OES + g * 4 * OES;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            if (dt * 32 + r4 * 8 >= dv_valid) continue;  // dv = 16: the upper half of the tile does not exist
            elem4 o4;
#pragma unroll
            for (int i = 0; i < 4; ++i) o4[i] = (elem)(oacc[dt][qt][r4 * 4 + i] * oscale);
            *(elem4*)(op + (dt * 32 + r4 * 8) * OES) = o4;
        }
}

// dst[row][h][0..d) (dense, fp16) = src[row * rs + h * hs + 0..d) (fp32, strides in elements); 8 elements per thread.
static __global__ __launch_bounds__(256) void hstu_cast_f32_f16_kernel(const float* src, int64_t rs, int64_t hs, int64_t rows, int H,
                                                                int d, _Float16* dst) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // over rows * H * d / 8
    const int d8 = d >> 3;
    if (idx >= rows * H * d8) return;
    const int c = (int)(idx % d8);
    const int64_t rh = idx / d8;
    const int h = (int)(rh % H);
    const int64_t row = rh / H;
    const float* sp = src + row * rs + (int64_t)h * hs + c * 8;
    const f32x4_t a = *(const f32x4_t*)sp, b = *(const f32x4_t*)(sp + 4);
    f16x8_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        o[i] = (_Float16)a[i];
        o[4 + i] = (_Float16)b[i];
    }
    *(f16x8_t*)(dst + idx * 8) = o;
}

// The same store made row-contiguous: the wave first writes its 32 x DV output tile (16-bit elements) to its own
// LDS area `lds` (32 rows of DV*2 + 16 bytes; the pad spreads the rows over the banks), then reads it back 16
// bytes per lane, 16 (or 8, 4) lanes per row, so that one store instruction covers whole rows.  The direct
// store above touches 32 rows per instruction, 16 bytes in each, which is slow to issue.
// Only the wave itself touches `lds`; the caller makes sure nobody still reads what was there before.
template <class TT, int DT>
__device__ __forceinline__ void store_output_via_lds(const f32x16_t (&oacc)[DT][1], char* lds, char* o, int64_t orow0, int q0,
                                                     int nq, int64_t o_rs, int64_t o_hs, int h, int lane, float oscale) {
    typedef typename TT::out_elem elem;  // 16 bits
    typedef __attribute__((ext_vector_type(4))) elem elem4;
    constexpr int ROWB = DT * 64 + 16;    // bytes per LDS row
    constexpr int CHR = DT * 4;           // 16-byte chunks per output row
    constexpr int RPI = 64 / CHR;         // rows per store instruction
    const int l32 = lane & 31, g = lane >> 5;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            elem4 o4;
#pragma unroll
            for (int i = 0; i < 4; ++i) o4[i] = (elem)(oacc[dt][0][r4 * 4 + i] * oscale);
            *HSTU_LDS(elem4, lds + l32 * ROWB + (dt * 32 + r4 * 8 + g * 4) * 2) = o4;
        }
    const int chunk = lane % CHR, rsub = lane / CHR;
    char* op = o + ((orow0 + q0 + rsub) * o_rs + (int64_t)h * o_hs) * 2 + chunk * 16;
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
        const int row = i * RPI + rsub;
        const i32x4_t v = *HSTU_LDS(const i32x4_t, lds + row * ROWB + chunk * 16);
        if (q0 + row < nq) *(i32x4_t*)(op + (int64_t)i * RPI * o_rs * 2) = v;
    }
}

// Unscaled fp32 accumulators of one block of 32 query rows to partial[split][row][head][dv]; 16 bytes per store.
template <int DT, int QT>
__device__ __forceinline__ void store_partial(const f32x16_t (&oacc)[DT][QT], int qt, float* partial, int64_t orow0, int ql,
                                              int nq, int H, int h, int g) {
    if (ql >= nq) return;
    float* op = partial + ((orow0 + ql) * H + h) * (int64_t)(DT * 32) + g * 4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            f32x4_t o4;
#pragma unroll
            for (int i = 0; i < 4; ++i) o4[i] = oacc[dt][qt][r4 * 4 + i];
            *(f32x4_t*)(op + dt * 32 + r4 * 8) = o4;
        }
}

// out = oscale * (sum of the runs of the row's row block), rounded once; one thread per 4 consecutive dv.
// The thread finds its sequence (delta mode: row / delta; otherwise a binary search of the offsets), skips
// rows the forward kernel does not produce (past max_seq_len, or a sequence shorter than delta) and reads the
// number of runs that run 0 of its row block recorded.
template <class ELEM>
__global__ __launch_bounds__(256) void hstu_reduce_splits_kernel(const FwdParams p, int64_t total_q, int dv, int bm) {
    typedef __attribute__((ext_vector_type(4))) ELEM elem4;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // over total_q * H * dv / 4
    const int dv4 = dv >> 2;
    if (idx >= total_q * p.H * dv4) return;
    const int c = (int)(idx % dv4);
    const int64_t rh = idx / dv4;
    const int h = (int)(rh % p.H);
    const int64_t row = rh / p.H;
    auto offset = [&](int j) -> int64_t {
        return p.offsets_i64 ? ((const int64_t*)p.offsets)[j] : (int64_t)((const int*)p.offsets)[j];
    };
    int b, r;
    if (p.delta > 0) {
        b = (int)(row / p.delta);
        r = (int)(row - (int64_t)b * p.delta);
        int64_t n = offset(b + 1) - offset(b);
        if (n > p.max_seq_len) n = p.max_seq_len;
        if (n <= 0 || n < p.delta) return;
    } else {
        int lo = 0, hi = p.B;  // last b with offsets[b] <= row
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (offset(mid) <= row) lo = mid; else hi = mid;
        }
        b = lo;
        const int64_t start = offset(b);
        int64_t n = offset(b + 1) - start;
        if (n > p.max_seq_len) n = p.max_seq_len;
        if (row - start >= n) return;
        r = (int)(row - start);
    }
    const int runs = p.split_counts[(b * p.H + h) * p.num_mb + r / bm];
    f32x4_t acc = *(const f32x4_t*)(p.partial + idx * 4);
    for (int s = 1; s < runs; ++s) {
        const f32x4_t x = *(const f32x4_t*)(p.partial + s * p.partial_stride + idx * 4);
        acc += x;
    }
    elem4 o4;
    const float osc = output_scale(p, row);
#pragma unroll
    for (int i = 0; i < 4; ++i) o4[i] = (ELEM)(acc[i] * osc);
    *(elem4*)(p.o + (row * p.o_rs + (int64_t)h * p.o_hs) * 2 + c * 8) = o4;
}

// The same copy through a buffer descriptor: 16 bytes per lane from descriptor base + soffset (wave-uniform) + voffset
// (per lane) to LDS at lds_base + 16*lane.  The hardware checks soffset + voffset against the descriptor's size and
// writes ZEROS to LDS for a lane that lies beyond it (established with a probe on the MI355X: both offsets take part in
// the check), so a tile that reaches past the end of a sequence needs no clamping: with the size set to the
// sequence's rows, what follows them (the next sequence, or nothing) is never read.  Issuing a copy costs no vector
// arithmetic and no 64-bit scalar arithmetic.
__device__ __forceinline__ i32x4_t make_buffer_rsrc(const char* base_uniform, unsigned bytes) {
    const uint64_t a = (uint64_t)uniform64((int64_t)(uintptr_t)base_uniform);
    i32x4_t r;
    r[0] = (int)(unsigned)a;
    r[1] = (int)((unsigned)(a >> 32) & 0xFFFFu);  // base[47:32]; stride 0: a raw buffer
    r[2] = (int)bytes;
    r[3] = 0x00020000;                            // 32-bit data format, no swizzle
    return r;
}
__device__ __forceinline__ void buffer_load_lds16(i32x4_t rsrc, unsigned voffset, unsigned soffset, const char* lds_base) {
    const unsigned m0 = (unsigned)(uintptr_t)HSTU_LDS(const char, lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(m0), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory");
}

// Same copy with the address split into a wave-uniform 64-bit base (scalar registers) and a 32-bit
// per-lane byte offset, so that issuing a copy costs no vector arithmetic.
__device__ __forceinline__ void global_load_lds16_soff(const char* base_uniform, unsigned lane_offset, const char* lds_base) {
    const unsigned m0 = (unsigned)(uintptr_t)HSTU_LDS(const char, lds_base);
    const uint64_t sbase = (uint64_t)uniform64((int64_t)(uintptr_t)base_uniform);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0), "v"(lane_offset), "s"(sbase)
                 : "memory");
}

// Copy `ROWS` rows of `ROWBYTES` bytes from global memory into LDS with the chunk swizzle.
// Rows at or beyond `n_rows_valid` re-read the last valid row (their products are masked).
template <int ROWS, int ROWBYTES, int NTHREADS, bool IS_V, int ES>
__device__ __forceinline__ void load_tile_to_lds(const char* gbase, int64_t row_stride_bytes, int row0,
                                                 int last_row, char* lds_tile, int wave, int lane) {
    constexpr int CH = ROWBYTES / 16;                // 16-byte chunks per row
    constexpr int INSTR = ROWS * CH / 64;            // wave-wide copies per tile
    constexpr int NWAVES = NTHREADS / 64;
#pragma unroll
    for (int i = 0; i < (INSTR + NWAVES - 1) / NWAVES; ++i) {
        int inst = wave + i * NWAVES;
        if (inst >= INSTR) break;  // narrow rows: fewer copies than waves
        int p = inst * 64 + lane;
        int row = p / CH;
        int phys = p % CH;
        int logical = phys ^ (IS_V ? swz_v<CH, ES>(row) : swz_k<CH>(row));
        int grow = row0 + row;
        grow = grow > last_row ? last_row : grow;
        const char* src = gbase + (int64_t)grow * row_stride_bytes + logical * 16;
        global_load_lds16(src, lds_tile + inst * 1024);
    }
}

}  // namespace hstu
