// Softmax attention over the paged cache whose heads talk to one another before the softmax.
//
// For a query at position i and a key at position j of the same request, inside the window
// (0 <= i - j < window, or every j <= i where window is 0):
//     raw_g    = scale * (q_g . k_kv(g),j) - slope_g * (i - j)            every query head g; slope may be absent
//     score_h  = sum_g talk[h][g] * raw_g                                 the heads' scores mixed; talk may be absent
//     weight_h = exp(score_h) / (sum over the window's j of exp(score_h) + exp(sink_h))
//     out_h    = sum_j weight_h v_kv(h),j
// The sink is a learned number per head that stands in the denominator once: it has no key, no value, no
// bias, and is not mixed.  Without it the denominator is the plain sum.
//
// A head's score needs every head's product with the same key, so a block takes ALL heads of one query
// token.  It walks the token's keys in chunks of 32 that are aligned to absolute positions: products of all
// (head, key) pairs into LDS, then the mixing and the running softmax with a half-wave per head, then the
// weighted sum of the values with the (head, value dim) pairs dealt out to the threads.  Scores, weights and
// sums are float whatever the cache's type.  The keys of a token can be dealt out to several blocks (parts
// of part_keys keys, aligned to absolute positions too); a second kernel then joins the parts and adds
// the sink.  What a token's result is depends on its own position and the window alone, never on the
// other rows of the step.
#include "common.h"
#include "api.h"
#include "recordable.h"

#define AM_CHUNK 32
#define AM_THREADS 256
#define AM_MAX_LDS (64 * 1024)

struct AttnMixed {
    const int* positions; const int* tok_seq; const int* block_table; int max_blocks;
    int nh; float scale; int window;
    const float* slopes; const float* talk; const float* sink;
    int part_keys, n_parts;          // part_keys 0: one block takes all keys of a token and finishes it
    float* part_acc; float* part_ml; // [n][parts][nh][hd] and [n][parts][nh][2] (running maximum, sum)
};

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> {
    bf16x8 v;
    __device__ __forceinline__ void load(const bf16_t* p) { v = *(const bf16x8*)p; }
    __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
};
template <> struct Vec8<float> {
    f32x4 a, b;
    __device__ __forceinline__ void load(const float* p) { a = *(const f32x4*)p; b = *(const f32x4*)(p + 4); }
    __device__ __forceinline__ float get(int i) const { return i < 4 ? a[i] : b[i - 4]; }
};

// ACC: (head, dim) pairs of the weighted sum per thread; nh * hd <= AM_THREADS * ACC
template <typename T, int ACC>
__global__ __launch_bounds__(AM_THREADS) void attn_mixed_kernel(const T* __restrict__ q, T* __restrict__ out, PagedCache cache,
                                                                AttnMixed a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int nh = a.nh, hd = cache.head_dim, ps = cache.page_size;
    float* qs = lds;                          // [nh][hd]
    float* raw = qs + nh * hd;                // [nh][CHUNK]
    float* pw = raw + nh * AM_CHUNK;          // [nh][CHUNK]
    float* tk = pw + nh * AM_CHUNK;           // [nh][nh]
    float* hm = tk + nh * nh;                 // running maximum per head
    float* hl = hm + nh;                      // running sum
    float* hc = hl + nh;                      // this chunk's correction of what was summed before
    float* hs = hc + nh;                      // slope
    const int token = blockIdx.x, tid = threadIdx.x;
    const int p = a.positions[token];
    const int* table = a.block_table + (size_t)a.tok_seq[token] * a.max_blocks;
    const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
    int k0 = lo, k1 = p;
    if (a.part_keys > 0) {
        const int part = lo / a.part_keys + blockIdx.y;
        k0 = max(lo, part * a.part_keys);
        k1 = min(p, (part + 1) * a.part_keys - 1);
    }
    const int group = nh / cache.n_kv_heads;
    {
        // a padding row of a fixed-size batch has no page, not even for its own position: zeros, and no key is read
        const int own = table[p / ps];
        if (own < 0 || own >= cache.n_pages) {
            if (a.part_keys > 0) {
                float* pm = a.part_ml + ((size_t)token * a.n_parts + blockIdx.y) * nh * 2;
                for (int h = tid; h < nh; h += AM_THREADS) { pm[2 * h] = -INFINITY; pm[2 * h + 1] = 0.f; }
            } else {
                for (int o = tid; o < nh * hd; o += AM_THREADS) out[(size_t)token * nh * hd + o] = from_f32<T>(0.f);
            }
            return;
        }
    }
    for (int e = tid; e < nh * hd; e += AM_THREADS) qs[e] = to_f32(q[(size_t)token * nh * hd + e]);
    for (int e = tid; e < nh * nh; e += AM_THREADS) tk[e] = a.talk ? a.talk[e] : 0.f;
    for (int e = tid; e < nh; e += AM_THREADS) {
        hm[e] = -INFINITY;
        hl[e] = 0.f;
        hs[e] = a.slopes ? a.slopes[e] : 0.f;
    }
    float acc[ACC];
#pragma unroll
    for (int u = 0; u < ACC; ++u) acc[u] = 0.f;
    __syncthreads();
    const T* base_ptr = (const T*)cache.base;
    for (int base = (k0 / AM_CHUNK) * AM_CHUNK; base <= k1; base += AM_CHUNK) {
        // ---- the products of every head with every key of the chunk
        for (int e = tid; e < nh * AM_CHUNK; e += AM_THREADS) {
            const int g = e / AM_CHUNK, j = base + (e % AM_CHUNK);
            float s = 0.f;
            if (j >= k0 && j <= k1) {
                const int page = min(max(table[j / ps], 0), cache.n_pages - 1);      // (a key inside the window always has a page)
                const T* kr = base_ptr + cache_k_offset(cache, page, g / group, j % ps, 0);
                const float* qg = qs + g * hd;
                float s0 = 0.f, s1 = 0.f;
                for (int d = 0; d < hd; d += 8) {
                    Vec8<T> kv;
                    kv.load(kr + d);
#pragma unroll
                    for (int i = 0; i < 8; i += 2) {
                        s0 = fmaf(qg[d + i], kv.get(i), s0);
                        s1 = fmaf(qg[d + i + 1], kv.get(i + 1), s1);
                    }
                }
                s = (s0 + s1) * a.scale - hs[g] * (float)(p - j);
            }
            raw[e] = s;
        }
        __syncthreads();
        // ---- mixing, and the running softmax of every head (a half-wave per head: its 32 lanes are the chunk's keys)
        for (int e0 = 0; e0 < nh * AM_CHUNK; e0 += AM_THREADS) {
            const int e = e0 + tid;
            const bool in = e < nh * AM_CHUNK;
            const int h = in ? e / AM_CHUNK : 0, jj = e % AM_CHUNK, j = base + jj;
            const bool valid = in && j >= k0 && j <= k1;
            float s;
            if (a.talk) {
                s = 0.f;
                for (int g = 0; g < nh; ++g) s = fmaf(tk[h * nh + g], raw[g * AM_CHUNK + jj], s);
            } else {
                s = raw[h * AM_CHUNK + jj];
            }
            if (!valid) s = -INFINITY;
            float top = s;
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, FL_WAVE));
            const float m_old = hm[h];
            const float m_new = fmaxf(m_old, top);
            const float pe = valid ? expf(s - m_new) : 0.f;
            float sum = pe;
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off, FL_WAVE);
            if (in) pw[e] = pe;
            if (in && jj == 0) {
                const float corr = m_old == -INFINITY ? 0.f : expf(m_old - m_new);    // (m_new is finite wherever a key was seen)
                hc[h] = m_new == -INFINITY ? 1.f : corr;
                hl[h] = hl[h] * (m_new == -INFINITY ? 1.f : corr) + sum;
                hm[h] = m_new;
            }
        }
        __syncthreads();
        // ---- the weighted sum of the values: eight keys of one value dim lie side by side in a page
#pragma unroll
        for (int u = 0; u < ACC; ++u) {
            const int o = tid + AM_THREADS * u;
            if (o >= nh * hd) continue;
            const int h = o / hd, d = o - h * hd;
            float sum = acc[u] * hc[h];
            const float* ph = pw + h * AM_CHUNK;
            if (ps % 8 == 0) {
                for (int j8 = 0; j8 < AM_CHUNK; j8 += 8) {
                    const int j = base + j8;
                    if (j + 7 < k0 || j > k1) continue;
                    const int page = min(max(table[j / ps], 0), cache.n_pages - 1);
                    Vec8<T> vv;
                    vv.load(base_ptr + cache_v_offset(cache, page, h / group, j % ps, d));
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const float w = ph[j8 + i];
                        if (w != 0.f) sum = fmaf(w, vv.get(i), sum);          // (a key outside the range may hold anything)
                    }
                }
            } else {
                for (int jj = 0; jj < AM_CHUNK; ++jj) {
                    const int j = base + jj;
                    const float w = ph[jj];
                    if (j < k0 || j > k1 || w == 0.f) continue;
                    sum = fmaf(w, to_f32(base_ptr[cache_v_offset(cache, min(max(table[j / ps], 0), cache.n_pages - 1), h / group, j % ps, d)]), sum);
                }
            }
            acc[u] = sum;
        }
        __syncthreads();
    }
    if (a.part_keys > 0) {
        float* pa = a.part_acc + ((size_t)token * a.n_parts + blockIdx.y) * nh * hd;
#pragma unroll
        for (int u = 0; u < ACC; ++u) {
            const int o = tid + AM_THREADS * u;
            if (o < nh * hd) pa[o] = acc[u];
        }
        float* pm = a.part_ml + ((size_t)token * a.n_parts + blockIdx.y) * nh * 2;
        for (int h = tid; h < nh; h += AM_THREADS) {
            pm[2 * h] = hm[h];
            pm[2 * h + 1] = hl[h];
        }
        return;
    }
#pragma unroll
    for (int u = 0; u < ACC; ++u) {
        const int o = tid + AM_THREADS * u;
        if (o >= nh * hd) continue;
        const int h = o / hd;
        // the sink joins the denominator; the larger of it and the running maximum is the reference point
        const float sk = a.sink ? a.sink[h] : -INFINITY;
        const float top = fmaxf(hm[h], sk);
        const float f = expf(hm[h] - top);
        const float den = hl[h] * f + (a.sink ? expf(sk - top) : 0.f);
        out[(size_t)token * nh * hd + o] = from_f32<T>(den > 0.f ? acc[u] * f / den : 0.f);
    }
}

// joins the parts of a token (rising order) and adds the sink: a thread per (token, head, dim)
template <typename T>
__global__ __launch_bounds__(AM_THREADS) void attn_mixed_join_kernel(T* __restrict__ out, AttnMixed a, int hd) {
    const int token = blockIdx.x, nh = a.nh;
    for (int o = threadIdx.x; o < nh * hd; o += AM_THREADS) {
        const int h = o / hd;
        const float* pm = a.part_ml + (size_t)token * a.n_parts * nh * 2;
        const float sk = a.sink ? a.sink[h] : -INFINITY;
        float top = sk;
        for (int part = 0; part < a.n_parts; ++part) top = fmaxf(top, pm[(part * nh + h) * 2]);
        float den = a.sink ? expf(sk - top) : 0.f, num = 0.f;
        for (int part = 0; part < a.n_parts; ++part) {
            const float m = pm[(part * nh + h) * 2], l = pm[(part * nh + h) * 2 + 1];
            if (!(l > 0.f)) continue;                                         // a part without keys
            const float f = expf(m - top);
            den = fmaf(l, f, den);
            num = fmaf(a.part_acc[((size_t)token * a.n_parts + part) * nh * hd + o], f, num);
        }
        out[(size_t)token * nh * hd + o] = from_f32<T>(den > 0.f ? num / den : 0.f);
    }
}

extern "C" int fl_attn_mixed_max_heads(int hd) {
    // what the block's LDS holds: q of all heads, two chunks of scores, the mixing matrix, four numbers per head
    int nh = 1;
    while (4 * ((nh + 1) * hd + 2 * (nh + 1) * AM_CHUNK + (nh + 1) * (nh + 1) + 4 * (nh + 1)) <= AM_MAX_LDS &&
           (nh + 1) * hd <= AM_THREADS * 64)
        ++nh;
    return nh;
}

extern "C" int fl_attn_mixed(const void* q, void* out, const void* cache_base, int dtype, const int* positions,
                             const int* tok_seq, const int* block_table, int max_blocks, int n, int nh, int nkv, int hd,
                             int page_size, int n_pages, float scale, int window, const float* slopes, const float* talk,
                             const float* sink, int part_keys, int n_parts, float* part_acc, float* part_ml,
                             hipStream_t stream) {
    FL_CHECK(n >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn_mixed: bad head counts %d/%d", nh, nkv);
    FL_CHECK(hd > 0 && hd % 8 == 0, "attn_mixed: heads are stored in multiples of 8 values, got %d", hd);
    FL_CHECK(window >= 0, "attn_mixed: negative window");
    FL_CHECK(nh <= fl_attn_mixed_max_heads(hd), "attn_mixed: %d heads of %d values are more than a block holds (%d)", nh, hd,
             fl_attn_mixed_max_heads(hd));
    FL_CHECK(part_keys >= 0 && part_keys % AM_CHUNK == 0, "attn_mixed: parts of %d keys (a multiple of %d wanted)", part_keys, AM_CHUNK);
    FL_CHECK(part_keys == 0 || (n_parts > 0 && n_parts <= 65535 && part_acc && part_ml), "attn_mixed: parts without their buffers");
    if (n == 0) return 0;
    PagedCache c{(void*)cache_base, nkv, page_size, hd, n_pages};
    AttnMixed a{positions, tok_seq, block_table, max_blocks, nh, scale, window, slopes, talk, sink,
                part_keys, part_keys ? n_parts : 1, part_acc, part_ml};
    const size_t lds = 4 * ((size_t)nh * hd + 2 * nh * AM_CHUNK + (size_t)nh * nh + 4 * nh);
    dim3 grid(n, a.n_parts);
    const int per_thread = ceil_div(nh * hd, AM_THREADS);
#define FL_AM(T, ACC) attn_mixed_kernel<T, ACC><<<grid, AM_THREADS, lds, stream>>>((const T*)q, (T*)out, c, a)
#define FL_AM_T(T)                       \
    do {                                 \
        if (per_thread <= 4) FL_AM(T, 4);        \
        else if (per_thread <= 16) FL_AM(T, 16); \
        else FL_AM(T, 64);               \
    } while (0)
    if (dtype == FL_F32) FL_AM_T(float);
    else if (dtype == FL_BF16) FL_AM_T(bf16_t);
    else FL_CHECK(false, "attn_mixed: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    if (part_keys > 0) {
        if (dtype == FL_F32) attn_mixed_join_kernel<float><<<n, AM_THREADS, 0, stream>>>((float*)out, a, hd);
        else attn_mixed_join_kernel<bf16_t><<<n, AM_THREADS, 0, stream>>>((bf16_t*)out, a, hd);
        FL_LAUNCH_CHECK();
    }
#undef FL_AM_T
#undef FL_AM
    return 0;
}
FL_RECORDABLE(fl_attn_mixed)
