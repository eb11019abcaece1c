/*
 * Scalar C restatement of HSTU jagged attention.  TEST INFRASTRUCTURE ONLY:
 * nothing shipped links or loads this file; tests use it to pin the PyTorch
 * oracle on small inputs.
 *
 * Follows generative_recommenders/ops/pytorch/pt_hstu_attention.py of the
 * reference: the arithmetic of pytorch_hstu_mha (lines 151, 167, 179, 182) and
 * pytorch_cached_hstu_mha (lines 227-250).  The mask of _get_valid_attn_mask
 * (lines 32-84) is deliberately NOT transcribed through its id formula: it is
 * written per position class (contextual / history / target row, explicit
 * column ranges), the way ops/cpp/hstu_attention/mask.h and
 * mainloop_fwd_sm90_tma_gmma_ws.h:629-697 of the reference state it, so that an
 * error in either formulation shows up as a disagreement.
 *
 * Position classes of a sequence of length n with c contextual positions and
 * t targets (u = n - t non-target positions):
 *     [0, c)  contextual      [c, u)  history      [u, n)  targets
 */
#include <math.h>
#include <stddef.h>

/* 1 if query position r may attend to key position s. t < 0 means "no targets given". */
static int valid_pair(int r, int s, int n, int c, int t, int w, int f) {
    int u = n - (t < 0 ? 0 : t);
    if (r < 0 || s < 0 || r >= n || s >= n) return 0;
    if (r == s) return 1;
    if (c > 0 && r < c) {
        /* contextual rows see every non-target position, past or future */
        return s < u;
    }
    if (s >= u) return 0;      /* nobody but itself sees a target */
    {
        /* r is a history or a target row; s is contextual or history */
        int row_pos = r < u ? r : u;            /* all targets sit at the same place: just after the history */
        int col_pos = (c > 0 && s < c) ? c - 1 : s; /* the contextual prefix counts as one position */
        int age = row_pos - col_pos;
        int window_off;
        if (age <= 0) return 0;                 /* causal */
        if (w <= 0) return 1;
        window_off = (f > 0) && (r >= u - f);    /* last f history rows and all targets ignore the window */
        return window_off || age <= w;
    }
}

void hstu_ref_mask(int n, int c, int t, int w, int f, unsigned char* out) {
    for (int r = 0; r < n; ++r)
        for (int s = 0; s < n; ++s) out[(size_t)r * n + s] = (unsigned char)valid_pair(r, s, n, c, t, w, f);
}

long long hstu_ref_count_pairs(int n, int c, int t, int w, int f, int delta_size) {
    long long cnt = 0;
    int r0 = delta_size > 0 ? n - delta_size : 0;
    for (int r = r0; r < n; ++r)
        for (int s = 0; s < n; ++s) cnt += valid_pair(r, s, n, c, t, w, f);
    return cnt;
}

/*
 * q: [Lq, H, Dqk]  k: [Lkv, H, Dqk]  v: [Lkv, H, Dv]  out: [Lq, H, Dv], all contiguous float.
 * delta_size == 0: q is jagged with the same offsets as k.
 * delta_size  > 0: q row b*delta_size + i is position n_b - delta_size + i of sequence b.
 * Returns 0, or -1 if a sequence is longer than max_seq_len or shorter than delta_size.
 */
int hstu_ref_fwd(const float* q, const float* k, const float* v, float* out, const long long* offsets,
                 const long long* num_targets, int B, int H, int Dqk, int Dv, int max_seq_len, float alpha,
                 int max_attn_len, int contextual_seq_len, int min_full_attn_seq_len, int delta_size) {
    for (int b = 0; b < B; ++b) {
        long long n = offsets[b + 1] - offsets[b];
        if (n > max_seq_len || n < delta_size) return -1;
    }
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int b = 0; b < B; ++b) {
        for (int h = 0; h < H; ++h) {
            long long s0 = offsets[b];
            int n = (int)(offsets[b + 1] - s0);
            int t = num_targets ? (int)num_targets[b] : -1;
            int r_first = delta_size > 0 ? n - delta_size : 0;
            for (int r = r_first; r < n; ++r) {
                long long qrow = delta_size > 0 ? (long long)b * delta_size + (r - r_first) : s0 + r;
                const float* qp = q + (qrow * H + h) * Dqk;
                float* op = out + (qrow * H + h) * Dv;
                double acc[1024];
                for (int d = 0; d < Dv; ++d) acc[d] = 0.0;
                for (int s = 0; s < n; ++s) {
                    if (!valid_pair(r, s, n, contextual_seq_len, t, max_attn_len, min_full_attn_seq_len)) continue;
                    const float* kp = k + ((s0 + s) * H + h) * Dqk;
                    const float* vp = v + ((s0 + s) * H + h) * Dv;
                    double dot = 0.0;
                    for (int d = 0; d < Dqk; ++d) dot += (double)qp[d] * (double)kp[d];
                    double x = dot * (double)alpha;
                    double p = x / (1.0 + exp(-x)) / (double)max_seq_len;
                    for (int d = 0; d < Dv; ++d) acc[d] += p * (double)vp[d];
                }
                for (int d = 0; d < Dv; ++d) op[d] = (float)acc[d];
            }
        }
    }
    return 0;
}
