/*
 * hstu_hip.h -- C ABI of libhstu_hip.so: HSTU jagged attention forward for gfx950 (MI355X).
 *
 * This is the boundary a caller binds instead of the reference's native operator
 * `hstu::hstu_mha_fwd` (generative_recommenders/ops/cpp/hstu_attention/flash_api_cpu.cpp:142-235,
 * host side flash_common.cpp:394-724).  Plain pointers and sizes only; no torch types.
 * All pointers are device pointers on the current HIP device.  Calls are asynchronous on the
 * stream given; nothing is allocated, nothing is read back to the host, no input is modified.
 *
 * Semantics (generative_recommenders/ops/pytorch/pt_hstu_attention.py:32-251):
 *     out[r] = sum_s M(r, s) * silu(alpha * <q_r, k_s>) / max_seq_len * v_s
 * per sequence b (rows seq_offsets[b] .. seq_offsets[b+1]) and head, where M is the
 * causal / max_attn_len / contextual_seq_len / num_targets mask of `_get_valid_attn_mask`.
 */
#ifndef HSTU_HIP_H_
#define HSTU_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types of q/k/v.  Output is the same type, except FP8_E4M3 inputs give BF16 output
 * (flash_common.cpp:596-607).
 * FP32 (accepted by the reference's PyTorch and Triton backends, hstu_attention_test.py:270-274; not by its native
 * op): the library first rounds q, k, v to fp16 copies in `workspace` (an 11-bit significand, one bit more than the
 * tf32 products of the reference's Triton path; magnitudes beyond 65504 overflow), runs the fp16 kernel and stores
 * the fp32 accumulators unrounded.  Needs the workspace, tile config 0 or 1, rows 16-byte aligned (strides multiples
 * of 4 elements). */
enum HstuDtype { HSTU_BF16 = 0, HSTU_FP16 = 1, HSTU_FP8_E4M3 = 2, HSTU_FP32 = 3 };

/* Status codes.  0 is success; the library never throws or aborts. */
enum HstuStatus {
    HSTU_OK = 0,
    HSTU_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
    HSTU_ERR_BAD_DTYPE = -2,      /* dtype not in HstuDtype (flash_common.cpp:428-441) */
    HSTU_ERR_BAD_HEAD_DIM = -3,   /* head dims this build has no kernel for (flash_common.cpp:591-594) */
    HSTU_ERR_MISALIGNED = -4,     /* base pointer or a stride breaks 16-byte row alignment (flash_common.cpp:447-452) */
    HSTU_ERR_BAD_SHAPE = -5,      /* negative / inconsistent sizes, max_seq_len <= 0, delta rows not B*delta */
    HSTU_ERR_UNSUPPORTED = -6,    /* legal in the reference but not built here */
    HSTU_ERR_LAUNCH = -7,         /* hipLaunchKernel failed; see hstu_hip_last_error() */
    HSTU_ERR_BAD_DEVICE = -8,     /* the current device is not gfx950 */
    HSTU_ERR_SCRATCH_LIMIT = -9,  /* hstu_hip_mha_fwd_noalloc: the call needs more than HSTU_NOALLOC_SCRATCH_BYTES */
    HSTU_ERR_BUSY = -10           /* hstu_hip_mha_fwd_noalloc: the device's scratch area is still in use by a call that was
                                     launched on another stream */
};

/*
 * Mirrors the subset of `Flash_fwd_params` (ops/cpp/hstu_attention/flash.h:24-110) that the
 * forward pass uses.  Strides are in ELEMENTS; the innermost (head-dim) stride is 1.
 */
typedef struct HstuFwdArgs {
    const void* q;            /* [total_q,  H, dqk]  (delta mode: [B*delta_size, H, dqk]) */
    const void* k;            /* [total_kv, H, dqk] */
    const void* v;            /* [total_kv, H, dv]  */
    void* out;                /* [total_q,  H, dv]  written for every row of every sequence */
    int64_t q_row_stride, q_head_stride;
    int64_t k_row_stride, k_head_stride;
    int64_t v_row_stride, v_head_stride;
    int64_t o_row_stride, o_head_stride;
    const void* seq_offsets;  /* [B+1] monotone, seq_offsets[0] == 0 */
    const void* num_targets;  /* [B] or NULL */
    int32_t seq_offsets_i64;  /* 1: int64 elements, 0: int32 (the reference's native op takes int32,
                                 flash_common.cpp:460-462; its Python callers pass int64) */
    int32_t num_targets_i64;
    int32_t batch;            /* B */
    int32_t heads;            /* H */
    int32_t dqk;              /* attention dim */
    int32_t dv;               /* value / output dim */
    int64_t total_q;          /* rows of q and out */
    int64_t total_kv;         /* rows of k and v */
    int32_t max_seq_len;      /* N: upper bound on every sequence length AND the 1/N output scale */
    int32_t delta_size;       /* 0: q is jagged like k.  >0: q holds the last delta_size positions
                                 of each sequence (pt_hstu_attention.py:190-251) */
    float alpha;
    int32_t max_attn_len;            /* 0 = unlimited */
    int32_t contextual_seq_len;      /* 0 = none */
    int32_t min_full_attn_seq_len;   /* 0 = none */
    int32_t dtype;                   /* HstuDtype */
    float q_scale, k_scale, v_scale; /* FP8 only: real value = stored value * scale (per tensor) */
    int32_t tile_config;             /* 0 = choose automatically; otherwise a value of hstu_hip_tile_configs() */
    int32_t sort_by_length;          /* scheduling hint of the reference (hstu_attention.py:115): start long
                                        sequences first.  Needs `workspace`; never changes the result */
    void* workspace;                 /* NULL, or device scratch of at least hstu_hip_workspace_bytes() bytes,
                                        4-byte aligned, owned by the caller, free to reuse once the call's work on
                                        `stream` has run */
    int64_t workspace_bytes;
    int32_t kv_splits;               /* 0 = choose automatically (delta mode with too few row blocks to fill and
                                        balance the chip is split when the workspace allows); 1 = never split;
                                        S = 2..8: cut the kv range of every row block into runs of
                                        ceil(ceil(max_seq_len / 64) / S) tiles of 64 rows, each run taken by its own
                                        workgroup, and add the fp32 partial results in a second kernel.  Needs
                                        `workspace`; tile configs 2 and 3 only.  The result is the same up to fp32
                                        summation order.  The reference has no such option: its kernels run one
                                        block per (sequence, head, row block) in both modes */
    const void* attn_scale;          /* NULL, or fp32 on the device: `attn_scale` of the reference
                                        (pt_hstu_attention.py:152-165; schema flash_api_cpu.cpp:142-235): silu(.) is
                                        multiplied by it INSTEAD of by 1 / max_seq_len.  One value for all rows
                                        (attn_scale_per_row = 0: the reference's 0-dim tensor) or one per query row,
                                        jagged like q ([total_q], attn_scale_per_row = 1).  Read on the device, never
                                        on the host.  Full form only (the reference's cached form does not take it) */
    int32_t attn_scale_per_row;
} HstuFwdArgs;

/* Library version, major*10000 + minor*100 + patch.  101: HstuFwdArgs gained attn_scale / attn_scale_per_row at its end
 * (a caller built against 100 passes a shorter struct and must be rebuilt). */
int hstu_hip_version(void);

/* Static, human-readable text for a status code. */
const char* hstu_hip_status_string(int status);

/* Text of the last HIP runtime error seen by this thread inside the library ("" if none). */
const char* hstu_hip_last_error(void);

/*
 * Validate `args` exactly as hstu_hip_mha_fwd would, without touching the device.
 * Replaces the TORCH_CHECKs of flash_common.cpp:420-594.
 */
int hstu_hip_check_args(const HstuFwdArgs* args);

/*
 * Launch the forward pass on `stream` (a hipStream_t; NULL = the default stream).
 * Replaces hstu::hstu_mha_fwd (flash_common.cpp:394-724) for both the full and the
 * delta-query (M-FALCON) forms.
 */
int hstu_hip_mha_fwd(const HstuFwdArgs* args, void* stream);

/*
 * Opt-in check of the caller contract, on the device (the library never reads the index arrays on the host): the
 * counterpart of the reference's debug-build checks (flash_common.cpp:529-541, HSTU_FLASH_ATTN_DEBUG_INFO).  Writes
 * four int32 to `report` (device memory) on `stream`: the number of sequences that break the contract, the index of the
 * first, a bit set of what is broken (1: offsets decrease, 2: longer than max_seq_len, 4: num_targets outside
 * [0, length], 8: fewer non-target positions than contextual_seq_len, 16: shorter than delta_size), and 1 if
 * seq_offsets[0] != 0 or seq_offsets[batch] != total_kv.  The forward pass itself never faults on such input, but rows
 * of an offending sequence may be left unwritten (longer than max_seq_len: the rows past it; shorter than delta_size:
 * all its rows) or masked as the formulas happen to give; the caller reads the report back when it wants to know.
 */
int hstu_hip_check_contract(const HstuFwdArgs* args, int32_t* report, void* stream);

/*
 * The same forward pass for callers that cannot allocate device memory: code under HIP graph capture, serving loops
 * with a fixed memory budget, harnesses that forbid hipMalloc.  No counterpart in the reference (its native op
 * allocates its tile semaphore and output itself, flash_common.cpp:596-678).  `args->workspace` is ignored: the scratch
 * memory hstu_hip_mha_fwd would take from it (work-item counters, sequence ranking, work lists, partial sums of a
 * kv-split) lives in a fixed area of HSTU_NOALLOC_SCRATCH_BYTES inside the library's device image, one per device,
 * held until the process ends.  The call allocates and frees nothing, on the device or through any library; the
 * caller still passes q, k, v, out and the index arrays.  Same kernels, same schedule and bit-identical results as
 * hstu_hip_mha_fwd given a workspace of hstu_hip_workspace_bytes(args).
 * Returns HSTU_ERR_SCRATCH_LIMIT (nothing launched; hstu_hip_last_error() names the two sizes) when
 * hstu_hip_workspace_bytes(args) exceeds the area -- FP32 inputs of more than a few million elements (their fp16
 * copies live there), kv-splits of very large delta batches, work lists of more than about 6 million row blocks.
 * All calls on one device share that device's area: two calls that may run at the same time on one device (different
 * streams) race on it and must be serialised by the caller; calls on one stream are safe back to back.  The library
 * catches the common form of the mistake without synchronising anything: it records an event behind every call and
 * returns HSTU_ERR_BUSY (nothing launched) when a call arrives on a DIFFERENT stream while the event of the call before
 * has not completed.  Under stream capture neither is possible (an event recorded into a graph cannot be queried), so
 * the check is skipped there and the caller's discipline is all there is.  Nothing needs clearing between calls (every
 * word a kernel reads was written earlier in the same call).  The first call on a device looks the area's address up
 * (hipGetSymbolAddress) and creates that event; make that call outside a capture.
 */
#define HSTU_NOALLOC_SCRATCH_BYTES (48u << 20)
int hstu_hip_mha_fwd_noalloc(const HstuFwdArgs* args, void* stream);

/*
 * Bytes of `workspace` the call would use with these arguments (0 if it needs none).  The library never
 * allocates: the reference's native op allocates its tile semaphore itself (flash_common.cpp:668-678);
 * here the caller passes scratch memory, or NULL to run without the options that need it.
 */
size_t hstu_hip_workspace_bytes(const HstuFwdArgs* args);

/*
 * The tile configuration and number of kv runs hstu_hip_mha_fwd would use for these arguments (either pointer may
 * be NULL).  Returns what hstu_hip_check_args returns.  Diagnostic only: the reference picks its tile configuration
 * with an autotuner at run time (ops/triton/triton_hstu_attention.py:1643), this library by a fixed rule.
 */
int hstu_hip_plan(const HstuFwdArgs* args, int32_t* tile_config, int32_t* kv_splits);

/* Number of selectable tile configurations and a short name for each (1-based ids). */
int hstu_hip_tile_configs(void);
const char* hstu_hip_tile_config_name(int id);

/*
 * ---- Backward of the full (non-delta) form ----
 *
 * dq, dk, dv from dout for the call described by `args` (its `out`, `tile_config`, `kv_splits` are ignored;
 * `delta_size` must be 0; bf16 or fp16).  Replaces triton_hstu_attention_bwd
 * (ops/triton/triton_hstu_attention.py:2825-2932, called from _AttentionFunction.backward, :3031-3093) and the
 * native hstu_mha_bwd (ops/cpp/hstu_attention/flash_common.cpp:726 onwards).  Nothing from the forward call is
 * needed except its inputs: the scores are recomputed.  Every row of dq / dk / dv that belongs to a sequence is
 * written; no atomics, so the result is bit-identical from run to run.  The gradients have the layout rules of
 * q / k / v: 16-byte aligned base, row and head strides in elements and multiples of 8, innermost stride 1.
 * `sort_by_length` (a scheduling hint: long sequences first) takes effect when `args->workspace` holds at least
 * 4 * batch bytes.  `args->attn_scale` must be NULL (HSTU_ERR_UNSUPPORTED otherwise): the gradients are those of the
 * 1 / max_seq_len scale; for a forward call that was given an attn_scale, multiply dout row by row by
 * attn_scale * max_seq_len first (the factor is per query row and commutes with everything behind it).
 *
 * Two ways to form dq.  Without more workspace than that, a second kernel recomputes the scores and dP from the query
 * side (seven matrix products for the five the mathematics needs).  With a 256-byte aligned workspace of at least
 * hstu_hip_mha_bwd_workspace_bytes(args) bytes -- 2 bytes per (query row, head, key position up to max_seq_len rounded
 * up to 128), e.g. 17 GB for 128 sequences x 4096 rows x 4 heads -- the kernel that forms dk and dv also writes dS,
 * rounded to the input type as the products use it, and dq is one streamed product dS K (HBM-bound; about a quarter
 * less time in total).  The two differ only by the rounding of the pre-scaled operand (q or k) of the score product.
 * The workspace need not be initialised and holds nothing of use afterwards.
 */
size_t hstu_hip_mha_bwd_workspace_bytes(const HstuFwdArgs* args);

typedef struct HstuBwdGrads {
    const void* dout;  /* [total_q, H, dv] */
    void* dq;          /* [total_q, H, dqk] */
    void* dk;          /* [total_kv, H, dqk] */
    void* dv;          /* [total_kv, H, dv] */
    int64_t do_row_stride, do_head_stride;
    int64_t dq_row_stride, dq_head_stride;
    int64_t dk_row_stride, dk_head_stride;
    int64_t dv_row_stride, dv_head_stride;
} HstuBwdGrads;

int hstu_hip_mha_bwd(const HstuFwdArgs* args, const HstuBwdGrads* grads, void* stream);

/*
 * ---- The data format either side of the path: per-batch concatenation of two jagged 2-D tensors ----
 *
 * `left`, `right` and `joined` are row-major [rows, row_bytes] byte matrices with row strides in BYTES; batch b owns
 * rows offsets[b] .. offsets[b+1] of a side, or exactly max_len rows when that side's offsets pointer is NULL
 * ("dense"); `joined` holds, for every batch, the left rows followed by the right rows, batch b starting at row
 * offsets_left[b] + offsets_right[b].  Caller contract as in the reference: per-batch lengths do not exceed
 * max_len_left / max_len_right (beyond that the reference's own result is ill-defined -- its mask then selects padding
 * rows -- and this library leaves the joined rows past max_len_left + max_len_right unwritten).
 * Replaces `concat_2D_jagged` / `split_2D_jagged` (generative_recommenders/ops/jagged_tensors.py:55-111; semantics
 * ops/pytorch/pt_jagged_tensors.py:31-173), which the reference uses to build cache (+) delta K/V for
 * `delta_hstu_mha` and to cut the cache out again (modules/stu.py:84-173).
 */
typedef struct HstuJaggedCopyArgs {
    void* left;                /* [total_left, row_bytes]   input of concat, output of split */
    void* right;               /* [total_right, row_bytes] */
    void* joined;              /* [total_left + total_right, row_bytes]   output of concat, input of split */
    int64_t left_row_stride, right_row_stride, joined_row_stride;  /* bytes, >= row_bytes */
    int64_t row_bytes;
    const void* offsets_left;  /* [B+1] or NULL */
    const void* offsets_right; /* [B+1] or NULL */
    int32_t offsets_left_i64, offsets_right_i64;  /* 1: int64 elements, 0: int32 */
    int32_t batch;
    int32_t max_len_left, max_len_right;
    int64_t total_left, total_right;  /* rows of `left` and `right` (for validation only) */
} HstuJaggedCopyArgs;

/* left, right -> joined.  Asynchronous on `stream`; allocates nothing. */
int hstu_hip_concat_2d_jagged(const HstuJaggedCopyArgs* args, void* stream);
/* joined -> left, right. */
int hstu_hip_split_2d_jagged(const HstuJaggedCopyArgs* args, void* stream);

/*
 * In-place form of the cache (+) delta concatenation: joined[offsets[b+1] - tail_len + i] = tail[b * tail_len + i]
 * for i < tail_len.  A K/V cache kept as "history rows, then tail_len spare rows" per sequence, with
 * offsets = kv_caching_offsets + tail_len * arange(B+1) (exactly the offsets `_construct_full_kv` returns,
 * modules/stu.py:133-173), then needs only the new rows copied per call instead of the whole history.  The
 * reference has no such entry point; it re-concatenates.  Strides in bytes; every sequence must hold at least
 * tail_len rows (shorter ones are left untouched).
 */
int hstu_hip_jagged_write_tail(void* joined, int64_t joined_row_stride, const void* offsets, int32_t offsets_i64,
                               const void* tail, int64_t tail_row_stride, int64_t row_bytes, int32_t batch,
                               int32_t tail_len, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_HIP_H_ */
