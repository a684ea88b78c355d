// Linear recurrences with a matrix state per head, token by token, and what prepares their inputs.
//
// fl_linear_scan: per request and head the state S [D][Dv] (float, in the request's slot between
// steps, zero when the slot is claimed).  For every token, with a decay g (one per head, or one per
// token and head), q and k of the head's query/key head and v of the head:
//     S <- g S
//     u = beta (v - S^T k)     (the delta rule; without beta: u = v)
//     S <- S + k u^T
//     o = S^T q                (the read-out sees the token's own write)
// The walk IS the recurrence, so a prompt cut anywhere leaves the same state and the same outputs.
//
// fl_conv_prepare: a short causal convolution over time per channel with silu behind it, for the
// channels of q, k and v side by side; the inputs of the last taps - 1 tokens of a request live in
// its slot (zeros before its start).  Then q and k are made unit vectors per head (q also times a
// factor), and the decay and write strength of every (token, head) are formed:
//     g = exp(-exp(A_log) softplus(a + dt_bias)),  beta = sigmoid(b).
// fl_conv_state_update moves the window of kept inputs on, after every block of the first has read it.
//
// fl_rotate_scale: rotation of the first dims of every head of two float row sets (q and k of a
// mixer that keeps no keys), each times a factor of its own afterwards.
#include "common.h"
#include "api.h"
#include "recordable.h"
#include "lanes.h"

#define LS_GROUP 16          // threads that share a column of S; they own the rows d = g, g + 16, ...
#define LS_COLS 16           // columns of S per block
#define LS_MAX_ROWS 32       // rows per thread: D <= LS_GROUP * LS_MAX_ROWS
#define LS_MAX_TAPS 16
#define LS_QK_REGS 8          // values of a q or k head per lane in the kernel that prepares them: D <= 512

// Block = (columns j0 .. j0 + 15, head, request); thread (g, c) holds S[d][j0 + c] for its RPT rows
// d = g * RPT .. g * RPT + RPT - 1 (neighbours, so that its q and k come from LDS in 16-byte reads).
// State of a head: S column by column, S[d][j] at j * D + d.
// The step's tokens come through LDS a run of RUN tokens at a time, rows 16 * RPT wide and zero behind D;
// the next run's values are asked for (into registers) before the walk over this run begins and put into
// LDS after it, so that the trip to memory hides behind the walk.
// MODE 0: a decay per head or per token and head, u = v; 1: the delta rule; 2: a decay per token, head AND key dim
// (`k` holds the forget gates f; the key is 1 - f: what is forgotten makes room for what is written); 3: the delta rule
// with a decay per token, head and key dim (`chan_decay`, rows ldc wide, heads x D: S <- diag(g) S before the correction)
template <int RPT, int MODE>
__global__ __launch_bounds__(LS_GROUP * LS_COLS) void linear_scan_kernel(
    const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, const float* __restrict__ v, int ldv,
    const float* __restrict__ head_decay, const float* __restrict__ tok_decay, const float* __restrict__ beta, int ldg,
    float* __restrict__ state, size_t slot_stride, const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
    const int* __restrict__ seq_slots, float* __restrict__ out, int H, int G, int D, int Dv,
    const float* __restrict__ chan_decay = nullptr, int ldc = 0) {
    constexpr int NT = LS_GROUP * LS_COLS;
    constexpr int DP = LS_GROUP * RPT;                                // a row of q or k in LDS
    constexpr int RUN = RPT <= 8 ? 32 : RPT <= 16 ? 16 : 8;          // tokens per run
    constexpr int PRE = RUN * DP / NT;                                // q (and k) values of a run per thread
    constexpr int PRE_V = (RUN * LS_COLS + NT - 1) / NT;
    const int g = threadIdx.x & (LS_GROUP - 1), c = threadIdx.x / LS_GROUP;
    const int j = blockIdx.x * LS_COLS + c, head = blockIdx.y, s = blockIdx.z;
    const int qk_head = head / (H / G);
    const bool live = j < Dv;
    const int start = seq_q_start[s], len = seq_q_len[s];
    float* st = state + (size_t)seq_slots[s] * slot_stride + (size_t)head * D * Dv;
    float S[RPT];
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int d = g * RPT + u;
        S[u] = (live && d < D) ? st[(size_t)j * D + d] : 0.f;
    }
    const float fixed = head_decay ? head_decay[head] : 1.f;
    __shared__ __attribute__((aligned(16))) float qs[RUN * DP];
    __shared__ __attribute__((aligned(16))) float ks[RUN * DP];
    __shared__ float vs[RUN * LS_COLS], fs[RUN * 2];
    __shared__ __attribute__((aligned(16))) float gs[MODE == 3 ? RUN * DP : 4];
    float pq[PRE], pk[PRE], pd[MODE == 3 ? PRE : 1], pv[PRE_V], pf0 = 0.f, pf1 = 0.f;
    auto fetch = [&](int t0) {                     // the values of the run that starts at token t0, into registers
        const int cnt = min(RUN, len - t0);
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int e = threadIdx.x + NT * i;
            const int tt = e / DP, d = e % DP;
            const bool in = tt < cnt && d < D;
            const size_t row = (size_t)(start + t0 + (in ? tt : 0));
            pq[i] = in ? q[row * ldq + qk_head * D + d] : 0.f;
            pk[i] = in ? k[row * ldk + qk_head * D + d] : (MODE == 2 ? 1.f : 0.f);
            if (MODE == 3) pd[i] = in ? chan_decay[row * ldc + head * D + d] : 1.f;
        }
#pragma unroll
        for (int i = 0; i < PRE_V; ++i) {
            const int e = threadIdx.x + NT * i;
            const int tt = e / LS_COLS, jj = blockIdx.x * LS_COLS + (e - tt * LS_COLS);
            pv[i] = (tt < cnt && jj < Dv) ? v[(size_t)(start + t0 + tt) * ldv + head * Dv + jj] : 0.f;
        }
        if (threadIdx.x < cnt) {
            const size_t row = (size_t)(start + t0 + threadIdx.x);
            pf0 = (MODE != 3 && tok_decay) ? tok_decay[row * ldg + head] : fixed;
            pf1 = (MODE == 1 || MODE == 3) ? beta[row * ldg + head] : 1.f;
        }
    };
    if (len > 0) fetch(0);
    for (int t0 = 0; t0 < len; t0 += RUN) {
        const int cnt = min(RUN, len - t0);
        __syncthreads();                           // the walk over the run before has read its last value
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            qs[threadIdx.x + NT * i] = pq[i];
            ks[threadIdx.x + NT * i] = pk[i];
            if (MODE == 3) gs[threadIdx.x + NT * i] = pd[i];
        }
#pragma unroll
        for (int i = 0; i < PRE_V; ++i)
            if (threadIdx.x + NT * i < RUN * LS_COLS) vs[threadIdx.x + NT * i] = pv[i];
        if (threadIdx.x < RUN) { fs[2 * threadIdx.x] = pf0; fs[2 * threadIdx.x + 1] = pf1; }
        __syncthreads();
        if (t0 + RUN < len) fetch(t0 + RUN);
#pragma unroll 2
        for (int tt = 0; tt < cnt; ++tt) {
            const float decay = fs[2 * tt];
            float uv = vs[tt * LS_COLS + c];
            float kr[RPT], qr[RPT];
#pragma unroll
            for (int u = 0; u < RPT; ++u) {
                kr[u] = ks[tt * DP + g * RPT + u];
                qr[u] = qs[tt * DP + g * RPT + u];
                if (MODE == 2) {
                    S[u] *= kr[u];
                    kr[u] = 1.0f - kr[u];
                } else if (MODE == 3) {
                    S[u] *= gs[tt * DP + g * RPT + u];
                } else {
                    S[u] *= decay;
                }
            }
            if (MODE == 1 || MODE == 3) {
                float seen0 = 0.f, seen1 = 0.f;                   // two chains of half the length
#pragma unroll
                for (int u = 0; u < RPT; u += 2) {
                    seen0 = fmaf(S[u], kr[u], seen0);
                    if (u + 1 < RPT) seen1 = fmaf(S[u + 1], kr[u + 1], seen1);
                }
                uv = fs[2 * tt + 1] * (uv - row_sum16(seen0 + seen1));
            }
            float num0 = 0.f, num1 = 0.f;
#pragma unroll
            for (int u = 0; u < RPT; u += 2) {
                S[u] = fmaf(kr[u], uv, S[u]);
                num0 = fmaf(S[u], qr[u], num0);
                if (u + 1 < RPT) {
                    S[u + 1] = fmaf(kr[u + 1], uv, S[u + 1]);
                    num1 = fmaf(S[u + 1], qr[u + 1], num1);
                }
            }
            const float num = row_sum16(num0 + num1);             // the 16 threads of a column are a row of lanes
            if (live && g == 0) out[((size_t)(start + t0 + tt) * H + head) * Dv + j] = num;
        }
    }
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
        const int d = g * RPT + u;
        if (live && d < D) st[(size_t)j * D + d] = S[u];
    }
}

extern "C" int fl_linear_scan_max_dim(void) { return LS_GROUP * LS_MAX_ROWS; }

static int linear_scan_launch(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                              const float* head_decay, const float* tok_decay, const float* beta, int ldg, float* state,
                              long slot_stride, const int* seq_q_start, const int* seq_q_len, const int* seq_slots,
                              float* out, int n_seqs, int H, int G, int D, int Dv, bool channel_decay, hipStream_t stream,
                              const float* chan_decay = nullptr, int ldc = 0) {
    FL_CHECK(!chan_decay || (beta && !head_decay && !tok_decay && !channel_decay && ldc >= H * D),
             "linear_scan: a decay per key dim under the delta rule comes with write strengths and without another decay");
    FL_CHECK(n_seqs >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0, "linear_scan: bad sizes");
    FL_CHECK(D <= LS_GROUP * LS_MAX_ROWS, "linear_scan: %d key dims per head, at most %d", D, LS_GROUP * LS_MAX_ROWS);
    FL_CHECK(ldq >= G * D && ldk >= G * D && ldv >= H * Dv, "linear_scan: rows narrower than their heads");
    FL_CHECK(chan_decay || (channel_decay ? (!head_decay && !tok_decay && !beta && H == G)
                                          : (!head_decay != !tok_decay)), "linear_scan: one decay per head, or one per token and head, or one per token, head and key dim");
    FL_CHECK((!tok_decay && !beta) || ldg >= H, "linear_scan: gate rows %d wide for %d heads", ldg, H);
    FL_CHECK(slot_stride >= (long)H * D * Dv, "linear_scan: a slot of %ld floats does not hold %d heads", slot_stride, H);
    if (n_seqs == 0) return 0;
    FL_CHECK(n_seqs <= 65535 && H <= 65535, "linear_scan: %d requests of %d heads are more than one grid takes", n_seqs, H);
    dim3 grid(ceil_div(Dv, LS_COLS), H, n_seqs);
    const int rpt = ceil_div(D, LS_GROUP);
#define FL_LS2(R, MODE)                                                                                               \
    linear_scan_kernel<R, MODE><<<grid, LS_GROUP * LS_COLS, 0, stream>>>(q, ldq, k, ldk, v, ldv, head_decay, tok_decay, beta, \
                                                                          ldg, state, (size_t)slot_stride, seq_q_start,        \
                                                                          seq_q_len, seq_slots, out, H, G, D, Dv, chan_decay, ldc)
#define FL_LS(R)             \
    do {                     \
        if (chan_decay) FL_LS2(R, 3);    \
        else if (channel_decay) FL_LS2(R, 2); \
        else if (beta) FL_LS2(R, 1);     \
        else FL_LS2(R, 0);               \
    } while (0)
    if (rpt <= 1) FL_LS(1);
    else if (rpt <= 2) FL_LS(2);
    else if (rpt <= 4) FL_LS(4);
    else if (rpt <= 8) FL_LS(8);
    else if (rpt <= 16) FL_LS(16);
    else FL_LS(LS_MAX_ROWS);
#undef FL_LS
#undef FL_LS2
    FL_LAUNCH_CHECK();
    return 0;
}

extern "C" int fl_linear_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                              const float* head_decay, const float* tok_decay, const float* beta, int ldg, float* state,
                              long slot_stride, const int* seq_q_start, const int* seq_q_len, const int* seq_slots,
                              float* out, int n_seqs, int H, int G, int D, int Dv, hipStream_t stream) {
    return linear_scan_launch(q, ldq, k, ldk, v, ldv, head_decay, tok_decay, beta, ldg, state, slot_stride, seq_q_start,
                              seq_q_len, seq_slots, out, n_seqs, H, G, D, Dv, false, stream);
}
FL_RECORDABLE(fl_linear_scan)

// The same walk with a forget gate per token, head and key dim: S <- diag(f) S + (1 - f) v^T, o = S^T q.
extern "C" int fl_linear_scan_channel(const float* q, int ldq, const float* f, int ldf, const float* v, int ldv, float* state,
                                      long slot_stride, const int* seq_q_start, const int* seq_q_len, const int* seq_slots,
                                      float* out, int n_seqs, int H, int D, int Dv, hipStream_t stream) {
    return linear_scan_launch(q, ldq, f, ldf, v, ldv, nullptr, nullptr, nullptr, 0, state, slot_stride, seq_q_start,
                              seq_q_len, seq_slots, out, n_seqs, H, H, D, Dv, true, stream);
}
FL_RECORDABLE(fl_linear_scan_channel)

// The delta rule with a decay per token, head and key dim: S <- diag(g) S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q.
// decay: rows ldd wide, heads x D; beta: rows ldb wide, one per head.
extern "C" int fl_linear_scan_delta_channel(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                            const float* decay, int ldd, const float* beta, int ldb, float* state,
                                            long slot_stride, const int* seq_q_start, const int* seq_q_len,
                                            const int* seq_slots, float* out, int n_seqs, int H, int G, int D, int Dv,
                                            hipStream_t stream) {
    FL_CHECK(decay && beta, "linear_scan_delta_channel: decays and write strengths are both needed");
    return linear_scan_launch(q, ldq, k, ldk, v, ldv, nullptr, nullptr, beta, ldb, state, slot_stride, seq_q_start,
                              seq_q_len, seq_slots, out, n_seqs, H, G, D, Dv, false, stream, decay, ldd);
}
FL_RECORDABLE(fl_linear_scan_delta_channel)

// g[t][h][d] = exp(-exp(A_log[h]) * softplus(a[t][col + h * D + d] + dt_bias[h * D + d])): the decays of a recurrence
// that forgets per head and key dim
__global__ __launch_bounds__(256) void channel_decay_kernel(const float* __restrict__ a, int ld, int col, const float* __restrict__ a_log,
                                                            const float* __restrict__ dt_bias, float* __restrict__ out, int H, int D) {
    const int t = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
    if (e >= H * D) return;
    const float z = a[(size_t)t * ld + col + e] + dt_bias[e];
    const float sp = z > 20.f ? z : log1pf(expf(z));
    out[(size_t)t * H * D + e] = expf(-expf(a_log[e / D]) * sp);
}

extern "C" int fl_channel_decay(const float* a, int ld, int col, const float* a_log, const float* dt_bias, float* out,
                                int n, int H, int D, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && D > 0 && col >= 0 && ld >= col + H * D, "channel_decay: columns %d..%d of rows %d wide", col, col + H * D, ld);
    if (n == 0) return 0;
    FL_CHECK(n <= 65535, "channel_decay: %d rows are more than one grid takes", n);
    channel_decay_kernel<<<dim3(ceil_div(H * D, 256), n), 256, 0, stream>>>(a, ld, col, a_log, dt_bias, out, H, D);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_channel_decay)

// out[t][f] = sum_r x[t][col + r] * wt[r][f] for a short run of r (the second factor of a projection of low rank, given
// TRANSPOSED, [rank][features], so that neighbouring threads read neighbouring values): x float rows, wt in its
// storage type, float sums in rising order of r
#define LR_TOKENS 8           // tokens a block of fl_lowrank_expand takes: a value of wt is read once for all of them
#define LR_FEW 16             // up to this many tokens a thread reads its feature's own row of the factor as it is stored
// (a step of few tokens: a block per token and 256 features, a thread walks the R neighbouring values of its feature's
// row, which the compiler fetches some at a time; the sums run in rising order of r as in the kernel below)
template <typename T>
__global__ __launch_bounds__(256) void lowrank_expand_rows_kernel(const float* __restrict__ x, int ld, int col, const T* __restrict__ w,
                                                                  float* __restrict__ out, int N, int R) {
    extern __shared__ float xr[];
    const int t = blockIdx.y;
    for (int r = threadIdx.x; r < R; r += 256) xr[r] = x[(size_t)t * ld + col + r];
    __syncthreads();
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f >= N) return;
    const T* wr = w + (size_t)f * R;
    float s = 0.f;
    for (int r = 0; r < R; ++r) s = fmaf(xr[r], to_f32(wr[r]), s);
    out[(size_t)t * N + f] = s;
}

template <typename T>
__global__ __launch_bounds__(256) void lowrank_expand_kernel(const float* __restrict__ x, int ld, int col, const T* __restrict__ w,
                                                             float* __restrict__ out, int n, int N, int R) {
    extern __shared__ float xr[];                         // [LR_TOKENS][R]
    const int t0 = blockIdx.y * LR_TOKENS, cnt = min(LR_TOKENS, n - t0);
    for (int e = threadIdx.x; e < LR_TOKENS * R; e += 256) {
        const int tt = e / R, r = e - tt * R;
        xr[e] = tt < cnt ? x[(size_t)(t0 + tt) * ld + col + r] : 0.f;
    }
    __syncthreads();
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f >= N) return;
    float s[LR_TOKENS];
#pragma unroll
    for (int tt = 0; tt < LR_TOKENS; ++tt) s[tt] = 0.f;
#pragma unroll 8
    for (int r = 0; r < R; ++r) {
        const float wv = to_f32(w[(size_t)r * N + f]);
#pragma unroll
        for (int tt = 0; tt < LR_TOKENS; ++tt) s[tt] = fmaf(xr[tt * R + r], wv, s[tt]);
    }
#pragma unroll
    for (int tt = 0; tt < LR_TOKENS; ++tt)
        if (tt < cnt) out[(size_t)(t0 + tt) * N + f] = s[tt];
}

extern "C" int fl_lowrank_expand(const float* x, int ld, int col, const void* w_rows, const void* w, int dtype, float* out,
                                 int n, int N, int R, hipStream_t stream) {
    FL_CHECK(n >= 0 && N > 0 && R > 0 && R <= 1024 && col >= 0 && ld >= col + R, "lowrank_expand: columns %d..%d of rows %d wide (a rank of at most 1024)", col, col + R, ld);
    FL_CHECK(w_rows && w, "lowrank_expand: the factor is wanted as it is stored and transposed");
    if (n == 0) return 0;
    if (n <= LR_FEW) {
        dim3 grid(ceil_div(N, 256), n);
        if (dtype == FL_F32) lowrank_expand_rows_kernel<float><<<grid, 256, R * sizeof(float), stream>>>(x, ld, col, (const float*)w_rows, out, N, R);
        else if (dtype == FL_BF16) lowrank_expand_rows_kernel<bf16_t><<<grid, 256, R * sizeof(float), stream>>>(x, ld, col, (const bf16_t*)w_rows, out, N, R);
        else FL_CHECK(false, "lowrank_expand: unknown dtype %d", dtype);
        FL_LAUNCH_CHECK();
        return 0;
    }
    dim3 grid(ceil_div(N, 256), ceil_div(n, LR_TOKENS));
    FL_CHECK(grid.y <= 65535, "lowrank_expand: %d rows are more than one grid takes", n);
    const size_t lds = (size_t)LR_TOKENS * R * sizeof(float);
    if (dtype == FL_F32) lowrank_expand_kernel<float><<<grid, 256, lds, stream>>>(x, ld, col, (const float*)w, out, n, N, R);
    else if (dtype == FL_BF16) lowrank_expand_kernel<bf16_t><<<grid, 256, lds, stream>>>(x, ld, col, (const bf16_t*)w, out, n, N, R);
    else FL_CHECK(false, "lowrank_expand: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_lowrank_expand)

// What stands between the joined projection of a mixer with forget gates per key dim and its walk:
// q = silu(q), f = lower + (1 - lower) * sigmoid(f + bias), both float, value by value.
__global__ __launch_bounds__(256) void forget_gates_kernel(const float* __restrict__ proj, int ld, int col_q, int col_f,
                                                           const float* __restrict__ bias, const float* __restrict__ lower,
                                                           float* __restrict__ q_out, float* __restrict__ f_out, int HD) {
    const float* row = proj + (size_t)blockIdx.x * ld;
    const int i = blockIdx.y * 256 + threadIdx.x;          // (a value per thread: a step of few tokens still fills units)
    if (i < HD) {
        const float zq = row[col_q + i];
        q_out[(size_t)blockIdx.x * HD + i] = zq / (1.0f + expf(-zq));
        const float low = lower ? lower[i] : 0.f;
        const float zf = row[col_f + i] + (bias ? bias[i] : 0.f);
        f_out[(size_t)blockIdx.x * HD + i] = low + (1.0f - low) / (1.0f + expf(-zf));
    }
}

extern "C" int fl_forget_gates(const float* proj, int ld, int col_q, int col_f, const float* bias, const float* lower,
                               float* q_out, float* f_out, int n, int HD, hipStream_t stream) {
    FL_CHECK(n >= 0 && HD > 0 && ld >= col_q + HD && ld >= col_f + HD && col_q >= 0 && col_f >= 0, "forget_gates: columns beyond rows %d wide", ld);
    if (n == 0) return 0;
    forget_gates_kernel<<<dim3(n, (HD + 255) / 256), 256, 0, stream>>>(proj, ld, col_q, col_f, bias, lower, q_out, f_out, HD);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_forget_gates)

// ------------------------------------------------------------------ short convolution, unit vectors, gates
struct ConvPrepare {
    const float* proj; int ld; int col0, col_b, col_a;
    const float* conv_w;                 // [C][taps], the last column is the current token's
    const float* a_log; const float* dt_bias;
    const float* conv_state; size_t slot_stride;      // per slot [taps - 1][C]: the inputs before the step, oldest first
    const int* tok_seq; const int* seq_q_start; const int* seq_slots;
    float* prep; float* gates;           // [n][C], [n][2 H]: decay, beta
    int G, H, D, Dv, taps;
    float q_scale, unit_eps;
};

// A wave per (token, head of q, k or v): a lane takes the head's channels lane, lane + 64, ...; the heads of a
// token are spread over blocks of four waves, so that a step of few tokens still fills units.
__global__ __launch_bounds__(256) void conv_prepare_kernel(ConvPrepare a) {
    const int token = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int C = 2 * a.G * a.D + a.H * a.Dv, taps = a.taps;
    const int s = a.tok_seq[token];
    const int back = token - a.seq_q_start[s];            // tokens of the request in this step before this one
    const float* hist = a.conv_state + (size_t)a.seq_slots[s] * a.slot_stride;
    float* dst = a.prep + (size_t)token * C;
    if (blockIdx.y == 0 && threadIdx.x < a.H) {
        const int h = threadIdx.x;
        const float* row = a.proj + (size_t)token * a.ld;
        if (a.a_log) {                                   // (null: the decays are formed elsewhere, only the write strengths here)
            const float z = row[a.col_a + h] + a.dt_bias[h];
            const float sp = z > 20.f ? z : log1pf(expf(z));
            a.gates[(size_t)token * 2 * a.H + h] = expf(-expf(a.a_log[h]) * sp);
        }
        a.gates[(size_t)token * 2 * a.H + a.H + h] = 1.0f / (1.0f + expf(-row[a.col_b + h]));
    }
    const int unit = blockIdx.y * 4 + wave;
    if (unit >= 2 * a.G + a.H) return;
    const bool is_qk = unit < 2 * a.G;
    const int width = is_qk ? a.D : a.Dv;
    const int c0 = is_qk ? unit * a.D : 2 * a.G * a.D + (unit - 2 * a.G) * a.Dv;
    auto convolved = [&](int c) {
        float y = 0.f;
        for (int jj = taps - 1; jj >= 0; --jj) {          // oldest input first
            const float x = jj <= back ? a.proj[(size_t)(token - jj) * a.ld + a.col0 + c]
                                       : hist[(size_t)(taps - 1 - (jj - back)) * C + c];
            y = fmaf(a.conv_w[(size_t)c * taps + (taps - 1 - jj)], x, y);
        }
        return y / (1.0f + expf(-y));
    };
    if (!is_qk) {
        for (int d = lane; d < width; d += 64) dst[c0 + d] = convolved(c0 + d);
        return;
    }
    // q and k heads become unit vectors (D <= 64 * LS_QK_REGS, checked on the host)
    float r[LS_QK_REGS];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < LS_QK_REGS; ++j) {
        const int d = lane + 64 * j;
        r[j] = d < width ? convolved(c0 + d) : 0.f;
        ss = fmaf(r[j], r[j], ss);
    }
    const float f = (unit < a.G ? a.q_scale : 1.f) / sqrtf(wave_sum(ss) + a.unit_eps);
#pragma unroll
    for (int j = 0; j < LS_QK_REGS; ++j)
        if (lane + 64 * j < width) dst[c0 + lane + 64 * j] = r[j] * f;
}

// per (request, channel): the kept inputs move on by the request's tokens of this step
__global__ __launch_bounds__(256) void conv_state_update_kernel(const float* __restrict__ proj, int ld, int col0, int C, int taps,
                                                                float* __restrict__ conv_state, size_t slot_stride,
                                                                const int* __restrict__ seq_q_start,
                                                                const int* __restrict__ seq_q_len,
                                                                const int* __restrict__ seq_slots) {
    const int c = blockIdx.x * 256 + threadIdx.x, s = blockIdx.y;
    if (c >= C) return;
    const int start = seq_q_start[s], len = seq_q_len[s], keep = taps - 1;
    float* hist = conv_state + (size_t)seq_slots[s] * slot_stride;
    float old[LS_MAX_TAPS];
#pragma unroll
    for (int r = 0; r < LS_MAX_TAPS; ++r) old[r] = r < keep ? hist[(size_t)r * C + c] : 0.f;
#pragma unroll
    for (int r = 0; r < LS_MAX_TAPS; ++r) {
        if (r >= keep) break;
        const int rel = len - keep + r;                    // which of this step's tokens, or (negative) an older one
        hist[(size_t)r * C + c] = rel >= 0 ? proj[(size_t)(start + rel) * ld + col0 + c] : old[r + len];
    }
}

extern "C" int fl_conv_max_taps(void) { return LS_MAX_TAPS; }

extern "C" int fl_conv_prepare(const float* proj, int ld, int col0, int col_b, int col_a, const float* conv_w,
                               const float* a_log, const float* dt_bias, float* conv_state, long slot_stride,
                               const int* tok_seq, const int* seq_q_start, const int* seq_q_len, const int* seq_slots,
                               float* prep, float* gates, int n, int n_seqs, int G, int H, int D, int Dv, int taps,
                               float q_scale, float unit_eps, hipStream_t stream) {
    FL_CHECK(n >= 0 && n_seqs >= 0 && G > 0 && H > 0 && D > 0 && Dv > 0, "conv_prepare: bad sizes");
    FL_CHECK(taps >= 1 && taps <= LS_MAX_TAPS, "conv_prepare: %d taps, at most %d", taps, LS_MAX_TAPS);
    FL_CHECK(H <= 256, "conv_prepare: %d heads, at most 256", H);
    const int C = 2 * G * D + H * Dv;
    FL_CHECK(ld >= col0 + C && ld >= col_b + H && (!a_log || ld >= col_a + H), "conv_prepare: columns beyond rows %d wide", ld);
    FL_CHECK(slot_stride >= (long)(taps - 1) * C, "conv_prepare: a slot of %ld floats does not hold %d inputs of %d channels",
             slot_stride, taps - 1, C);
    if (n == 0) return 0;
    FL_CHECK(n_seqs <= 65535, "conv_prepare: %d requests are more than one grid takes", n_seqs);
    ConvPrepare a{proj, ld, col0, col_b, col_a, conv_w, a_log, dt_bias, conv_state, (size_t)slot_stride, tok_seq, seq_q_start,
                  seq_slots, prep, gates, G, H, D, Dv, taps, q_scale, unit_eps};
    FL_CHECK(D <= 64 * LS_QK_REGS, "conv_prepare: %d key dims per head, at most %d", D, 64 * LS_QK_REGS);
    dim3 pgrid(n, ceil_div(2 * G + H, 4));
    FL_CHECK(pgrid.y <= 65535, "conv_prepare: %d heads are more than one grid takes", 2 * G + H);
    conv_prepare_kernel<<<pgrid, 256, 0, stream>>>(a);
    FL_LAUNCH_CHECK();
    if (taps > 1 && n_seqs > 0) {
        dim3 grid(ceil_div(C, 256), n_seqs);
        conv_state_update_kernel<<<grid, 256, 0, stream>>>(proj, ld, col0, C, taps, conv_state, (size_t)slot_stride, seq_q_start,
                                                           seq_q_len, seq_slots);
        FL_LAUNCH_CHECK();
    }
    return 0;
}
FL_RECORDABLE(fl_conv_prepare)

// ------------------------------------------------------------------ rotation of float rows
// out[t][h][d] of two row sets a (H heads) and b (H heads), both D wide per head: the first rot dims turned
// by the step's table, pairs (i, i + rot/2) or (2i, 2i + 1); a times scale_a, b times scale_b afterwards.
__global__ __launch_bounds__(256) void rotate_scale_kernel(const float* __restrict__ proj, int ld, int col_a, int col_b,
                                                           const float2* __restrict__ cs, int rot, int interleaved, float scale_a,
                                                           float scale_b, float* __restrict__ out_a, float* __restrict__ out_b,
                                                           int H, int D) {
    const size_t token = blockIdx.x;
    const int half = rot >> 1;
    for (int e = threadIdx.x; e < 2 * H * D; e += 256) {
        const bool is_b = e >= H * D;
        const int f = is_b ? e - H * D : e;
        const int h = f / D, d = f - h * D;
        const float* src = proj + token * ld + (is_b ? col_b : col_a) + h * D;
        float v = src[d];
        if (d < rot) {
            int i, partner;
            bool first;
            if (interleaved) { i = d >> 1; first = !(d & 1); partner = d ^ 1; }
            else { first = d < half; i = first ? d : d - half; partner = first ? d + half : d - half; }
            const float2 c = cs[token * half + i];
            const float o = src[partner];
            v = first ? v * c.x - o * c.y : v * c.x + o * c.y;
        }
        (is_b ? out_b : out_a)[token * H * D + f] = v * (is_b ? scale_b : scale_a);
    }
}

extern "C" int fl_rotate_scale(const float* proj, int ld, int col_a, int col_b, const float* cs, int rot, int interleaved,
                               float scale_a, float scale_b, float* out_a, float* out_b, int n, int H, int D,
                               hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && D > 0, "rotate_scale: bad sizes");
    FL_CHECK(rot >= 0 && rot <= D && rot % 2 == 0 && (rot == 0 || cs), "rotate_scale: rotated dims %d of head %d", rot, D);
    FL_CHECK(ld >= col_a + H * D && ld >= col_b + H * D, "rotate_scale: columns beyond rows %d wide", ld);
    if (n == 0) return 0;
    rotate_scale_kernel<<<n, 256, 0, stream>>>(proj, ld, col_a, col_b, (const float2*)cs, rot, interleaved, scale_a, scale_b,
                                               out_a, out_b, H, D);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_rotate_scale)
