// Hyper-connections: a residual stream kept in S copies, and what a sublayer does to them.
//
// The copies of a token lie side by side, xs[t][s][i] (float).  Around a sublayer with the learned numbers
// in[S], out[S] and mix[S][S] (indexed [from][to]):
//     u   = sum_s in[s] x_s                      what the sublayer's norm reads
//     x_t <- sum_s mix[s][t] x_s + out[t] * y    all copies at once from the old ones, y the sublayer's output
//                                                (plus y_bias, one value per column, where the sublayer's last product has a bias)
// fl_hyper_step does the second line for the sublayer that has just run (if y is given) and the first for the one
// that runs next (if `in` is given), in one pass over the copies: the new copies are written, their weighted sum u is
// kept in float (u_out) and, if a gain is given, normed in the same kernel:
//     normed = u / sqrt(mean(u^2) + eps) * gain      (the gain as it multiplies: one plus the stored weight, for a
//                                                     norm whose weight is stored around zero)
// `in` of ones and no gain gives the plain sum of the copies (what the model's last norm reads).
// fl_hyper_spread makes the S copies of the embedding's output.  All arithmetic is float; only `normed` is stored
// in the compute type.
#include "common.h"
#include "api.h"
#include "recordable.h"

#define HY_MAX_STREAMS 16

struct HyperStep {
    float* xs; int S, W;
    const float* y;                 // [n][W] or null: nothing is written
    const float* y_bias;            // [W] or null: added to every row of y as it is read (a bias of the sublayer's last product)
    const float* mix; const float* out_w;
    const float* in_w;              // [S] or null: nothing is read
    float* u_out;                   // [n][W] or null
    const float* gain; float eps;   // [W] or null
    const int* rows;                // picks the tokens that are read (one output row each), or null; only without y
};

// A block per token.  NT threads, each VEC neighbouring values of a row at a time (one 16-byte access where the width
// allows it); all copies of those values are asked for before the first is used.  The first KEEP turns of the walk over
// a row keep their u in registers for the norm (a row up to NT * VEC * KEEP wide is read once); what lies beyond is read
// back from u_out.  SMAX bounds the copies at compile time (4 or 16).  Rows of two thousand values or more take blocks of
// 1,024 threads, so that a row is a turn or two and a step of few rows is as long as one trip to memory and back.  The
// block's shape follows from the width alone, never from the step's rows: a row's bits do not depend on its neighbours.
template <typename T, int NT, int VEC, int KEEP, int SMAX>
__global__ __launch_bounds__(NT) void hyper_step_kernel(HyperStep a, T* __restrict__ normed) {
    __shared__ float coef[HY_MAX_STREAMS * HY_MAX_STREAMS + 2 * HY_MAX_STREAMS];
    __shared__ float lds[NT / 64];
    const int S = a.S, W = a.W;
    float* mixs = coef;                               // [from][to]
    float* outs = coef + HY_MAX_STREAMS * HY_MAX_STREAMS;
    float* ins = outs + HY_MAX_STREAMS;
    for (int e = threadIdx.x; e < S * S; e += NT) mixs[e] = a.y ? a.mix[e] : 0.f;
    for (int e = threadIdx.x; e < S; e += NT) {
        outs[e] = a.y ? a.out_w[e] : 0.f;
        ins[e] = a.in_w ? a.in_w[e] : 0.f;
    }
    __syncthreads();
    const int r = blockIdx.x;
    const int t = a.rows ? a.rows[r] : r;
    float* x = a.xs + (size_t)t * S * W;
    const float* yr = a.y ? a.y + (size_t)t * W : nullptr;
    float ss = 0.f;
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    // the values c .. c + VEC - 1 of every copy: write the new copies, return u
    auto turn = [&](int c) {
        vec_t old[SMAX];
#pragma unroll
        for (int s = 0; s < SMAX; ++s)
            if (s < S) old[s] = *(const vec_t*)(x + (size_t)s * W + c);
        vec_t u = 0.f;
        if (yr) {
            vec_t yv = *(const vec_t*)(yr + c);
            if (a.y_bias) yv += *(const vec_t*)(a.y_bias + c);
#pragma unroll
            for (int to = 0; to < SMAX; ++to) {
                if (to >= S) break;
                vec_t v = 0.f;
#pragma unroll
                for (int s = 0; s < SMAX; ++s)
                    if (s < S) v += mixs[s * S + to] * old[s];
                v += outs[to] * yv;
                *(vec_t*)(x + (size_t)to * W + c) = v;
                u += ins[to] * v;
            }
        } else {
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
                if (s < S) u += ins[s] * old[s];
        }
        return u;
    };
    vec_t kept[KEEP];
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int c = (k * NT + threadIdx.x) * VEC;
        kept[k] = 0.f;
        if (c >= W) continue;
        kept[k] = turn(c);
        if (a.in_w && a.u_out) *(vec_t*)(a.u_out + (size_t)r * W + c) = kept[k];
#pragma unroll
        for (int i = 0; i < VEC; ++i) ss = fmaf(kept[k][i], kept[k][i], ss);
    }
    for (int c = (KEEP * NT + threadIdx.x) * VEC; c < W; c += NT * VEC) {
        const vec_t u = turn(c);
        if (a.in_w && a.u_out) *(vec_t*)(a.u_out + (size_t)r * W + c) = u;
#pragma unroll
        for (int i = 0; i < VEC; ++i) ss = fmaf(u[i], u[i], ss);
    }
    if (!a.in_w || !a.gain) return;
    ss = block_sum<NT / 64>(ss, lds);                 // (the barrier inside also orders this block's u_out stores before its reads)
    const float inv = 1.0f / sqrtf(ss / (float)W + a.eps);
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int c = (k * NT + threadIdx.x) * VEC;
        if (c >= W) continue;
#pragma unroll
        for (int i = 0; i < VEC; ++i) normed[(size_t)r * W + c + i] = from_f32<T>(kept[k][i] * inv * a.gain[c + i]);
    }
    for (int c = (KEEP * NT + threadIdx.x) * VEC; c < W; c += NT * VEC)
#pragma unroll
        for (int i = 0; i < VEC; ++i) normed[(size_t)r * W + c + i] = from_f32<T>(a.u_out[(size_t)r * W + c + i] * inv * a.gain[c + i]);
}

#define HY_WIDE_ROW 2048      // from this many values a row a block has 1,024 threads

extern "C" int fl_hyper_step(float* xs, int n, int S, int W, const float* y, const float* y_bias, const float* mix, const float* out_w,
                             const float* in_w, const int* rows, int n_rows, float* u_out, const float* gain, float eps,
                             void* normed, int out_dtype, hipStream_t stream) {
    FL_CHECK(n >= 0 && S >= 1 && S <= HY_MAX_STREAMS && W > 0, "hyper_step: %d copies of %d values (at most %d copies)", S, W, HY_MAX_STREAMS);
    FL_CHECK(!y || (mix && out_w), "hyper_step: a sublayer's output without its numbers");
    FL_CHECK(y || !y_bias, "hyper_step: a bias without the output it belongs to");
    FL_CHECK(!gain || (in_w && u_out && normed), "hyper_step: a norm needs what it reads and where it writes");
    FL_CHECK(!rows || !y, "hyper_step: picked rows are read only");
    FL_CHECK(out_dtype == FL_F32 || out_dtype == FL_BF16, "hyper_step: unknown dtype %d", out_dtype);
    const int blocks = rows ? n_rows : n;
    if (blocks <= 0) return 0;
    HyperStep a{xs, S, W, y, y_bias, mix, out_w, in_w, u_out, gain, eps, rows};
    const bool few = W >= HY_WIDE_ROW, wide = W % 4 == 0, small = S <= 4;
#define FL_HY(T, NT, VEC, KEEP, SMAX) hyper_step_kernel<T, NT, VEC, KEEP, SMAX><<<blocks, NT, 0, stream>>>(a, (T*)normed)
#define FL_HY_S(T, NT, VEC, KEEP) do { if (small) FL_HY(T, NT, VEC, KEEP, 4); else FL_HY(T, NT, VEC, KEEP, HY_MAX_STREAMS); } while (0)
#define FL_HY_T(T)                                   \
    do {                                             \
        if (few && wide) FL_HY_S(T, 1024, 4, 2);     \
        else if (few) FL_HY_S(T, 1024, 1, 4);        \
        else if (wide) FL_HY_S(T, 256, 4, 4);        \
        else FL_HY_S(T, 256, 1, 8);                  \
    } while (0)
    if (out_dtype == FL_F32) FL_HY_T(float);
    else FL_HY_T(bf16_t);
#undef FL_HY_T
#undef FL_HY_S
#undef FL_HY
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_hyper_step)

// xs[t][s][:] = x[t][:] for every copy s
__global__ __launch_bounds__(256) void hyper_spread_kernel(const float* __restrict__ x, float* __restrict__ xs, int S, int W) {
    const int t = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= W) return;
    const float v = x[(size_t)t * W + i];
    for (int s = 0; s < S; ++s) xs[((size_t)t * S + s) * W + i] = v;
}

extern "C" int fl_hyper_spread(const float* x, float* xs, int n, int S, int W, hipStream_t stream) {
    FL_CHECK(n >= 0 && S >= 1 && W > 0, "hyper_spread: bad sizes");
    if (n == 0) return 0;
    FL_CHECK(n <= 65535, "hyper_spread: %d rows are more than one grid takes", n);
    hyper_spread_kernel<<<dim3(ceil_div(W, 256), n), 256, 0, stream>>>(x, xs, S, W);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_hyper_spread)

// out = ca * a + cb * b, value by value (two mixers side by side, each with a factor)
__global__ __launch_bounds__(256) void scaled_sum_kernel(const float* __restrict__ a, float ca, const float* __restrict__ b, float cb,
                                                         float* __restrict__ out, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) out[i] = ca * a[i] + cb * b[i];
}

extern "C" int fl_scaled_sum(const float* a, float ca, const float* b, float cb, float* out, long total, hipStream_t stream) {
    FL_CHECK(total >= 0, "scaled_sum: bad size");
    if (total == 0) return 0;
    scaled_sum_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(a, ca, b, cb, out, total);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_scaled_sum)

// x <- cap * tanh(x / cap), value by value (a soft cap on logits)
__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, long total, float cap) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int fl_softcap_inplace(float* x, long total, float cap, hipStream_t stream) {
    FL_CHECK(total >= 0 && cap > 0.f, "softcap: bad size or cap");
    if (total == 0) return 0;
    softcap_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(x, total, cap);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_softcap_inplace)
