// A feed-forward of routed experts: the router's choice, the experts' products over the rows each
// was given, and the sum per token.
//
//   fl_moe_route    (two kernels: the picks, a wave per token; then one block that counts and sorts)
//                   scores -> for every token its `top` experts (largest router logits, the lower index among
//                   equals) and their weights; the (token, expert) pairs sorted by expert, cut into row
//                   tiles that each belong to one expert
//   fl_moe_gemm     out[p] = (scale[p] * x[src[p]]) W_e^T for the sorted pairs p, e the expert of p's tile
//   fl_moe_combine  delta[t] = sum_k y[place of (t, k)]  (+ sigmoid(shared gate logit) * shared[t])
// Nothing of a step's values is read on the host: the lists live on the device and the grids are
// sized by their upper bounds (tiles that a step does not use end at once).
#include "common.h"
#include "api.h"
#include "recordable.h"

#define MOE_TILE 64           // rows of a tile of fl_moe_gemm
#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 16

// logits: float rows ld wide, the experts' at col0 .. col0 + E - 1.  kind 0: weight = sigmoid(logit);
// kind 1: weight = softmax over all experts; kind 2: softmax over the chosen logits only.  renorm: the chosen
// weights are divided by their sum (kind 2 always).
// place [n * top]: where pair (t, k) lies in the sorted order; src_row / src_scale [n * top]: token and weight
// of every sorted place; tiles [max_tiles][4] = (expert, first place, places, 0), expert -1: unused.
__global__ __launch_bounds__(256) void moe_pick_kernel(const float* __restrict__ logits, int ld, int col0, int n, int E,
                                                       int top, int kind, int renorm, int* __restrict__ place,
                                                       float* __restrict__ pair_w) {
    // a wave per token: the lanes hold the token's logits (lane, lane + 64, ...), and every rank is a best-of-wave
    // (the larger logit, the lower index among equals)
    const int lane = threadIdx.x & 63;
    const int nu = (E + 63) >> 6;
    for (int t = blockIdx.x * 4 + (threadIdx.x >> 6); t < n; t += gridDim.x * 4) {
        const float* z = logits + (size_t)t * ld + col0;
        float zv[MOE_MAX_EXPERTS / 64];
#pragma unroll
        for (int u = 0; u < MOE_MAX_EXPERTS / 64; ++u) zv[u] = (u < nu && lane + 64 * u < E) ? z[lane + 64 * u] : -INFINITY;
        float zmax = -INFINITY, zsum = 0.f;
        if (kind == 1) {
#pragma unroll
            for (int u = 0; u < MOE_MAX_EXPERTS / 64; ++u) if (u < nu) zmax = fmaxf(zmax, zv[u]);
            zmax = wave_max(zmax);
#pragma unroll
            for (int u = 0; u < MOE_MAX_EXPERTS / 64; ++u) zsum += (u < nu && lane + 64 * u < E) ? expf(zv[u] - zmax) : 0.f;
            zsum = wave_sum(zsum);
        }
        int chosen[MOE_MAX_TOP];
        float w[MOE_MAX_TOP], wsum = 0.f, zfirst = 0.f;
        for (int k = 0; k < top; ++k) {
            float bz = -INFINITY;
            int best = 0x7fffffff;
#pragma unroll
            for (int u = 0; u < MOE_MAX_EXPERTS / 64; ++u) {
                const int e = lane + 64 * u;
                if (u < nu && e < E && (zv[u] > bz || (zv[u] == bz && e < best)) && zv[u] > -INFINITY) { bz = zv[u]; best = e; }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float oz = __shfl_xor(bz, off, FL_WAVE);
                const int oe = __shfl_xor(best, off, FL_WAVE);
                if (oz > bz || (oz == bz && oe < best)) { bz = oz; best = oe; }
            }
            if (best == 0x7fffffff) {                              // (only logits of minus infinity are left: the lowest index not yet taken)
                best = 0;
                for (int e = 0; e < E; ++e) {
                    bool taken = false;
                    for (int u = 0; u < k; ++u) taken |= chosen[u] == e;
                    if (!taken) { best = e; break; }
                }
            }
#pragma unroll
            for (int u = 0; u < MOE_MAX_EXPERTS / 64; ++u)
                if (u < nu && lane + 64 * u == best) zv[u] = -INFINITY;      // taken
            chosen[k] = best;
            if (k == 0) zfirst = bz;                              // the largest logit
            w[k] = kind == 2 ? expf(bz - zfirst) : kind == 1 ? expf(bz - zmax) / zsum : 1.0f / (1.0f + expf(-bz));
            wsum += w[k];
        }
        if (lane == 0) {
            for (int k = 0; k < top; ++k) {
                place[(size_t)t * top + k] = chosen[k];
                pair_w[(size_t)t * top + k] = (renorm || kind == 2) ? w[k] / wsum : w[k];
            }
        }
    }
}

// The picks of a router whose choice and weights differ: s = softmax(z) over all E outputs; the choice goes by
// s + correction (correction may be null); the outputs form n_groups equal groups of neighbours, a group's score is
// its largest choice score, and only outputs of the keep_groups best groups (the lower index among equals) can be
// chosen; the weights are the chosen s divided by their sum (+ 1e-20) times scale.  A wave per token.
template <int NU>
__global__ __launch_bounds__(256) void moe_pick_grouped_kernel(const float* __restrict__ logits, int ld, int col0, int n, int E,
                                                               int top, const float* __restrict__ correction, int n_groups,
                                                               int keep_groups, float scale, int* __restrict__ place,
                                                               float* __restrict__ pair_w) {
    const int lane = threadIdx.x & 63;
    constexpr int nu = NU;                         // outputs per lane (lane, lane + 64, ...): E <= 64 * NU
    const int per = E / n_groups;
    for (int t = blockIdx.x * 4 + (threadIdx.x >> 6); t < n; t += gridDim.x * 4) {
        const float* z = logits + (size_t)t * ld + col0;
        float sv[NU], cv[NU];
        float zmax = -INFINITY, zsum = 0.f;
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            sv[u] = (u < nu && lane + 64 * u < E) ? z[lane + 64 * u] : -INFINITY;
            if (u < nu) zmax = fmaxf(zmax, sv[u]);
        }
        zmax = wave_max(zmax);
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            sv[u] = (u < nu && lane + 64 * u < E) ? expf(sv[u] - zmax) : 0.f;
            zsum += sv[u];
        }
        zsum = wave_sum(zsum);
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const int e = lane + 64 * u;
            sv[u] = sv[u] / zsum;
            cv[u] = (u < nu && e < E) ? sv[u] + (correction ? correction[e] : 0.f) : -INFINITY;
        }
        // best-of-wave over (value, index): the larger value, the lower index among equals
        auto best_of = [&](float& bz, int& best) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float oz = __shfl_xor(bz, off, FL_WAVE);
                const int oe = __shfl_xor(best, off, FL_WAVE);
                if (oz > bz || (oz == bz && oe < best)) { bz = oz; best = oe; }
            }
        };
        if (n_groups > 1 && keep_groups < n_groups) {
            // A group is kept if fewer than keep_groups groups beat it (a larger score, or an equal one at a lower index).
            // Every lane learns the scores of its own outputs' groups, then counts the groups that beat them; what lies
            // outside the kept groups can no longer be chosen.
            float own[NU];
            int beaten[NU];
#pragma unroll
            for (int u = 0; u < NU; ++u) { own[u] = -INFINITY; beaten[u] = 0; }
            for (int pass = 0; pass < 2; ++pass) {
                for (int g = 0; g < n_groups; ++g) {
                    float m = -INFINITY;
#pragma unroll
                    for (int u = 0; u < NU; ++u) {
                        const int e = lane + 64 * u;
                        if (u < nu && e < E && e / per == g) m = fmaxf(m, cv[u]);
                    }
                    m = wave_max(m);
#pragma unroll
                    for (int u = 0; u < NU; ++u) {
                        const int mine = (lane + 64 * u) / per;
                        if (pass == 0) {
                            if (mine == g) own[u] = m;
                        } else if (m > own[u] || (m == own[u] && g < mine)) {
                            ++beaten[u];
                        }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (beaten[u] >= keep_groups) cv[u] = -INFINITY;
        }
        int chosen[MOE_MAX_TOP];
        float w[MOE_MAX_TOP], wsum = 0.f;
        for (int k = 0; k < top; ++k) {
            float bz = -INFINITY;
            int best = 0x7fffffff;
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int e = lane + 64 * u;
                if (u < nu && e < E && cv[u] > -INFINITY && (cv[u] > bz || (cv[u] == bz && e < best))) { bz = cv[u]; best = e; }
            }
            best_of(bz, best);
            if (best == 0x7fffffff) {                              // (nothing is left to choose from: the lowest index not yet taken)
                best = 0;
                for (int e = 0; e < E; ++e) {
                    bool taken = false;
                    for (int u = 0; u < k; ++u) taken |= chosen[u] == e;
                    if (!taken) { best = e; break; }
                }
            }
            float sw = 0.f;
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (u < nu && lane + 64 * u == best) { sw = sv[u]; cv[u] = -INFINITY; }      // taken
            sw = wave_sum(sw);                                     // (one lane holds it)
            chosen[k] = best;
            w[k] = sw;
            wsum += sw;
        }
        if (lane == 0) {
            for (int k = 0; k < top; ++k) {
                place[(size_t)t * top + k] = chosen[k];
                pair_w[(size_t)t * top + k] = w[k] / (wsum + 1e-20f) * scale;
            }
        }
    }
}

// The (token, expert) pairs that moe_pick_kernel left (place[pair] = expert) counted, sorted by expert and cut into tiles.
// Outputs E_real .. E - 1 of the router are identity experts (no matrices): their tiles carry expert -1, which the
// products skip, and a 1 in the fourth place, which fl_moe_identity looks for.
__global__ __launch_bounds__(1024) void moe_route_kernel(int n, int E, int E_real, int top, int* __restrict__ place,
                                                         int* __restrict__ src_row, float* __restrict__ src_scale,
                                                         const float* __restrict__ pair_w, int* __restrict__ tiles, int max_tiles) {
    __shared__ int count[MOE_MAX_EXPERTS];
    __shared__ int first[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < E; e += 1024) count[e] = 0;
    __syncthreads();
    for (int a = threadIdx.x; a < n * top; a += 1024) atomicAdd(&count[place[a]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tile = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at;
            for (int r = 0; r < count[e] && tile < max_tiles; r += MOE_TILE, ++tile) {
                tiles[4 * tile + 0] = e < E_real ? e : -1;
                tiles[4 * tile + 1] = at + r;
                tiles[4 * tile + 2] = min(MOE_TILE, count[e] - r);
                tiles[4 * tile + 3] = e < E_real ? 0 : 1;
            }
            at += count[e];
            count[e] = 0;                      // from here on: places handed out
        }
        for (; tile < max_tiles; ++tile) {      // (unused)
            tiles[4 * tile + 0] = -1;
            tiles[4 * tile + 1] = tiles[4 * tile + 2] = tiles[4 * tile + 3] = 0;
        }
    }
    __syncthreads();
    // a token's pairs take the next free places of their experts; which of an expert's places a pair
    // gets changes nothing in its result (every row of the products is computed on its own)
    for (int a = threadIdx.x; a < n * top; a += 1024) {
        const int e = place[a];
        const int p = first[e] + atomicAdd(&count[e], 1);
        src_row[p] = a / top;
        src_scale[p] = pair_w[a];
        place[a] = p;
    }
}

extern "C" int fl_moe_tile_rows(void) { return MOE_TILE; }

extern "C" int fl_moe_route(const float* logits, int ld, int col0, int n, int E, int top, int kind, int renorm,
                            int* place, int* src_row, float* src_scale, float* pair_w, int* tiles, int max_tiles,
                            hipStream_t stream) {
    FL_CHECK(n >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= MOE_MAX_TOP && top <= E,
             "moe_route: %d of %d experts (at most %d of %d)", top, E, MOE_MAX_TOP, MOE_MAX_EXPERTS);
    FL_CHECK(ld >= col0 + E && col0 >= 0, "moe_route: columns %d..%d of rows %d wide", col0, col0 + E, ld);
    {
        const long pairs = (long)n * top;          // an expert's last tile may be short: pairs / 64 full tiles and one per expert at most
        FL_CHECK((long)max_tiles >= pairs / MOE_TILE + (pairs < E ? pairs : E), "moe_route: %d tiles cannot hold %ld rows of %d experts", max_tiles, pairs, E);
    }
    FL_CHECK(kind >= 0 && kind <= 2, "moe_route: unknown scoring %d", kind);
    if (n == 0) return 0;
    const int pick_blocks = n < 4 * 1024 ? (n + 3) / 4 : 1024;
    moe_pick_kernel<<<pick_blocks, 256, 0, stream>>>(logits, ld, col0, n, E, top, kind, renorm, place, pair_w);
    FL_LAUNCH_CHECK();
    moe_route_kernel<<<1, 1024, 0, stream>>>(n, E, E, top, place, src_row, src_scale, pair_w, tiles, max_tiles);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_moe_route)

// fl_moe_route for a router with a correction of the choice, groups of experts and identity experts (see
// moe_pick_grouped_kernel).  E counts all the router's outputs, the last n_identity of which are identity experts.
extern "C" int fl_moe_route_grouped(const float* logits, int ld, int col0, int n, int E, int n_identity, int top,
                                    const float* correction, int n_groups, int keep_groups, float scale, int* place,
                                    int* src_row, float* src_scale, float* pair_w, int* tiles, int max_tiles,
                                    hipStream_t stream) {
    FL_CHECK(n >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= MOE_MAX_TOP && top <= E,
             "moe_route_grouped: %d of %d experts (at most %d of %d)", top, E, MOE_MAX_TOP, MOE_MAX_EXPERTS);
    FL_CHECK(n_identity >= 0 && n_identity < E, "moe_route_grouped: %d identity experts among %d outputs", n_identity, E);
    FL_CHECK(n_groups >= 1 && E % n_groups == 0 && keep_groups >= 1 && keep_groups <= n_groups && keep_groups <= MOE_MAX_TOP &&
             keep_groups * (E / n_groups) >= top, "moe_route_grouped: %d of %d groups over %d outputs cannot give %d choices",
             keep_groups, n_groups, E, top);
    FL_CHECK(ld >= col0 + E && col0 >= 0, "moe_route_grouped: columns %d..%d of rows %d wide", col0, col0 + E, ld);
    {
        const long pairs = (long)n * top;
        FL_CHECK((long)max_tiles >= pairs / MOE_TILE + (pairs < E ? pairs : E), "moe_route_grouped: %d tiles cannot hold %ld rows of %d experts", max_tiles, pairs, E);
    }
    if (n == 0) return 0;
    const int pick_blocks = n < 4 * 1024 ? (n + 3) / 4 : 1024;
#define FL_PICK(NU) moe_pick_grouped_kernel<NU><<<pick_blocks, 256, 0, stream>>>(logits, ld, col0, n, E, top, correction, n_groups, keep_groups, scale, place, pair_w)
    if (E <= 64) FL_PICK(1);               // (a lane's outputs live in registers: as few slots as the router's width needs)
    else if (E <= 128) FL_PICK(2);
    else if (E <= 256) FL_PICK(4);
    else FL_PICK(MOE_MAX_EXPERTS / 64);
#undef FL_PICK
    FL_LAUNCH_CHECK();
    moe_route_kernel<<<1, 1024, 0, stream>>>(n, E, E - n_identity, top, place, src_row, src_scale, pair_w, tiles, max_tiles);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_moe_route_grouped)

// The rows of identity experts: y[p] = scale[p] * x[src[p]] for the places p of every tile that fl_moe_route_grouped
// marked as an identity expert's.
template <typename TIn>
__global__ __launch_bounds__(256) void moe_identity_kernel(const TIn* __restrict__ x, const int* __restrict__ src_row,
                                                           const float* __restrict__ src_scale, float* __restrict__ y,
                                                           const int* __restrict__ tiles, int W) {
    if (tiles[4 * blockIdx.y + 3] != 1) return;
    const int p0 = tiles[4 * blockIdx.y + 1], M = tiles[4 * blockIdx.y + 2];
    for (int r = 0; r < M; ++r) {
        const TIn* xr = x + (size_t)src_row[p0 + r] * W;
        const float f = src_scale[p0 + r];
        for (int c = blockIdx.x * 256 + threadIdx.x; c < W; c += 256 * gridDim.x) y[(size_t)(p0 + r) * W + c] = f * to_f32(xr[c]);
    }
}

extern "C" int fl_moe_identity(const void* x, int dtype, const int* src_row, const float* src_scale, float* y,
                               const int* tiles, int max_tiles, int W, hipStream_t stream) {
    FL_CHECK(max_tiles >= 0 && W > 0 && src_row && src_scale, "moe_identity: bad sizes or no rows");
    if (max_tiles == 0) return 0;
    FL_CHECK(max_tiles <= 65535, "moe_identity: %d row tiles are more than one grid takes", max_tiles);
    dim3 grid(min(ceil_div(W, 256), 16), max_tiles);
    if (dtype == FL_F32) moe_identity_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, src_row, src_scale, y, tiles, W);
    else if (dtype == FL_BF16) moe_identity_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, src_row, src_scale, y, tiles, W);
    else FL_CHECK(false, "moe_identity: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_moe_identity)

// The plain product (64 x 64 tile, 4 x 4 per thread, k in steps of 16, the steps' sums added with a
// compensated addition) over the rows of one tile of one expert.  src_row / src_scale may be null (the
// rows are then the sorted places themselves, unscaled).  A scaled row is rounded to the storage type
// before it is multiplied, as a stored activation would be.
template <typename TIn>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const TIn* __restrict__ x, const int* __restrict__ src_row,
                                                       const float* __restrict__ src_scale, const TIn* __restrict__ w,
                                                       float* __restrict__ out, const int* __restrict__ tiles, int N, int K) {
    __shared__ float xs[16][68];
    __shared__ float ws[16][68];
    __shared__ int rows_of[MOE_TILE];
    __shared__ float scale_of[MOE_TILE];
    const int e = tiles[4 * blockIdx.y + 0];
    if (e < 0) return;
    const int p0 = tiles[4 * blockIdx.y + 1], M = tiles[4 * blockIdx.y + 2];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int n0 = blockIdx.x * 64;
    const TIn* we = w + (size_t)e * N * K;
    if (threadIdx.x < MOE_TILE) {
        const int i = threadIdx.x;
        rows_of[i] = i < M ? (src_row ? src_row[p0 + i] : p0 + i) : 0;
        scale_of[i] = (i < M && src_scale) ? src_scale[p0 + i] : 1.0f;
    }
    __syncthreads();
    float acc[4][4], lost[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) { acc[i][j] = 0.f; lost[i][j] = 0.f; }
    for (int k0 = 0; k0 < K; k0 += 16) {
        for (int el = threadIdx.x; el < 1024; el += 256) {
            const int row = el >> 4, kk = el & 15;
            const int gk = k0 + kk, gn = n0 + row;
            float xv = 0.f;
            if (row < M && gk < K) {
                xv = to_f32(x[(size_t)rows_of[row] * K + gk]);
                if (src_scale) xv = to_f32(from_f32<TIn>(xv * scale_of[row]));
            }
            xs[kk][row] = xv;
            ws[kk][row] = (gn < N && gk < K) ? to_f32(we[(size_t)gn * K + gk]) : 0.f;
        }
        __syncthreads();
        float part[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) part[i][j] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float y = part[i][j] - lost[i][j];
                const float t = acc[i][j] + y;
                lost[i][j] = (t - acc[i][j]) - y;
                acc[i][j] = t;
            }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = ty * 4 + i;
        if (r >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn < N) out[(size_t)(p0 + r) * N + gn] = acc[i][j];
        }
    }
}

extern "C" int fl_moe_gemm(const void* x, int dtype, const int* src_row, const float* src_scale, const void* w,
                           float* out, const int* tiles, int max_tiles, int N, int K, hipStream_t stream) {
    FL_CHECK(max_tiles >= 0 && N > 0 && K > 0, "moe_gemm: bad sizes");
    if (max_tiles == 0) return 0;
    FL_CHECK(max_tiles <= 65535, "moe_gemm: %d row tiles are more than one grid takes", max_tiles);
    dim3 grid(ceil_div(N, 64), max_tiles);
    if (dtype == FL_F32)
        moe_gemm_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, src_row, src_scale, (const float*)w, out, tiles, N, K);
    else if (dtype == FL_BF16)
        moe_gemm_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, src_row, src_scale, (const bf16_t*)w, out, tiles, N, K);
    else
        FL_CHECK(false, "moe_gemm: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_moe_gemm)

// delta[t][c] = sum over k (rising) of y[place[t * top + k]][c], plus sigmoid(gate logit of t) * shared[t][c]
// where a shared expert is given (gate: float rows ldg wide, the logit at gate_col; null: ungated).
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, int top,
                                                          const float* __restrict__ shared, const float* __restrict__ gate,
                                                          int ldg, int gate_col, float* __restrict__ delta, int W) {
    const int t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= W) return;
    float v = 0.f;
    for (int k = 0; k < top; ++k) v += y[(size_t)place[(size_t)t * top + k] * W + c];
    if (shared) {
        const float g = gate ? 1.0f / (1.0f + expf(-gate[(size_t)t * ldg + gate_col])) : 1.0f;
        v += g * shared[(size_t)t * W + c];
    }
    delta[(size_t)t * W + c] = v;
}

extern "C" int fl_moe_combine(const float* y, const int* place, int top, const float* shared, const float* gate, int ldg,
                              int gate_col, float* delta, int n, int W, hipStream_t stream) {
    FL_CHECK(n >= 0 && W > 0 && top >= 0, "moe_combine: bad sizes");
    FL_CHECK(!gate || (gate_col >= 0 && ldg > gate_col), "moe_combine: gate column %d of rows %d wide", gate_col, ldg);
    if (n == 0) return 0;
    FL_CHECK(n <= 65535, "moe_combine: %d rows are more than one grid takes", n);
    dim3 grid(ceil_div(W, 256), n);
    moe_combine_kernel<<<grid, 256, 0, stream>>>(y, place, top, shared, gate, ldg, gate_col, delta, W);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_moe_combine)

// ------------------------------------------------------------------ activations of an ungated feed-forward
// kind 0: gelu with the error function, 0.5 z (1 + erf(z / sqrt 2)); 1: its tanh form,
// 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))); 2: silu, z / (1 + exp(-z)).
template <typename TOut>
__global__ __launch_bounds__(256) void activation_kernel(const float* __restrict__ x, TOut* __restrict__ out, long total, int kind,
                                                         const float* __restrict__ bias = nullptr, int width = 1) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const float z = bias ? x[i] + bias[i % width] : x[i];
    float y;
    if (kind == 0) y = 0.5f * z * (1.0f + erff(z * 0.70710678118654752440f));
    else if (kind == 1) y = 0.5f * z * (1.0f + tanhf(0.79788456080286535588f * (z + 0.044715f * z * z * z)));
    else if (kind == 3) y = z > 0.f ? z * z : 0.f;
    else y = z / (1.0f + expf(-z));
    out[i] = from_f32<TOut>(y);
}

extern "C" int fl_activation(const float* x, void* out, int out_dtype, long total, int kind, hipStream_t stream) {
    FL_CHECK(total >= 0 && kind >= 0 && kind <= 3, "activation: bad size or kind %d", kind);
    if (total == 0) return 0;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (out_dtype == FL_F32) activation_kernel<float><<<blocks, 256, 0, stream>>>(x, (float*)out, total, kind);
    else if (out_dtype == FL_BF16) activation_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (bf16_t*)out, total, kind);
    else FL_CHECK(false, "activation: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_activation)

// out[r][i] = act(x[r][i] + bias[i]): the activation of a feed-forward whose first product has a bias
extern "C" int fl_bias_activation(const float* x, const float* bias, void* out, int out_dtype, int n, int width, int kind,
                                  hipStream_t stream) {
    FL_CHECK(n >= 0 && width > 0 && kind >= 0 && kind <= 3 && bias, "bias_activation: bad size, kind %d or no bias", kind);
    const long total = (long)n * width;
    if (total == 0) return 0;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (out_dtype == FL_F32) activation_kernel<float><<<blocks, 256, 0, stream>>>(x, (float*)out, total, kind, bias, width);
    else if (out_dtype == FL_BF16) activation_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (bf16_t*)out, total, kind, bias, width);
    else FL_CHECK(false, "bias_activation: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_bias_activation)

// ------------------------------------------------------------------ re-entry of the residual stream
// out[r] = [a[r] ; b[r]] in the storage type (two float rows of W values side by side).
template <typename TOut>
__global__ __launch_bounds__(256) void concat_cast_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          TOut* __restrict__ out, int W) {
    const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= 2 * W) return;
    out[(size_t)r * 2 * W + c] = from_f32<TOut>(c < W ? a[(size_t)r * W + c] : b[(size_t)r * W + c - W]);
}

extern "C" int fl_concat_cast(const float* a, const float* b, void* out, int out_dtype, int n, int W, hipStream_t stream) {
    FL_CHECK(n >= 0 && W > 0, "concat_cast: bad sizes");
    if (n == 0) return 0;
    FL_CHECK(n <= 65535, "concat_cast: %d rows are more than one grid takes", n);
    dim3 grid(ceil_div(2 * W, 256), n);
    if (out_dtype == FL_F32) concat_cast_kernel<float><<<grid, 256, 0, stream>>>(a, b, (float*)out, W);
    else if (out_dtype == FL_BF16) concat_cast_kernel<bf16_t><<<grid, 256, 0, stream>>>(a, b, (bf16_t*)out, W);
    else FL_CHECK(false, "concat_cast: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_concat_cast)

// x[r][c] += v[c]
__global__ __launch_bounds__(256) void add_rowvec_kernel(float* __restrict__ x, const float* __restrict__ v, int W) {
    const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c < W) x[(size_t)r * W + c] += v[c];
}

extern "C" int fl_add_rowvec(float* x, const float* v, int n, int W, hipStream_t stream) {
    FL_CHECK(n >= 0 && W > 0, "add_rowvec: bad sizes");
    if (n == 0) return 0;
    FL_CHECK(n <= 65535, "add_rowvec: %d rows are more than one grid takes", n);
    dim3 grid(ceil_div(W, 256), n);
    add_rowvec_kernel<<<grid, 256, 0, stream>>>(x, v, W);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_add_rowvec)
