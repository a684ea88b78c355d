// Softmax attention over the paged cache whose heads talk to one another before the softmax.
//
// For a query at position i and a key at position j <= i of the same request that the mask lets through
// (window > 0: i - j < window; chunk > 0 instead: i and j in the same run of `chunk` positions counted from 0;
// neither: every j <= i; and, whatever the rest says, every j < keep_first: the first tokens stay visible):
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
    int nh; float scale; int window, keep_first, chunk;
    const float* slopes; const float* talk; const float* sink;
    int part_keys, n_parts;          // part_keys 0: one block takes all keys of a token and finishes it
    float* part_acc; float* part_ml; // [n][parts][nh][hd] and [n][parts][nh][2] (running maximum, sum)
};

// the first key that the window or the chunk of a query at position p lets through
__device__ __forceinline__ int am_mask_lo(const AttnMixed& a, int p) {
    return a.chunk > 0 ? p - p % a.chunk : a.window > 0 ? max(0, p - a.window + 1) : 0;
}

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
    const int lo = am_mask_lo(a, p);
    const int kept = min(a.keep_first, lo);          // the keys [0, kept) are seen beside [lo, p]; the first part's block takes them
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
    const int main_k0 = k0, main_k1 = k1;
    for (int range = 0; range < 2; ++range) {
    // two runs of keys: the kept first tokens (if the mask hides what follows them), then the window's or chunk's own
    if (range == 0) {
        if (kept <= 0 || (a.part_keys > 0 && blockIdx.y != 0)) continue;
        k0 = 0; k1 = kept - 1;
    } else {
        k0 = main_k0; k1 = main_k1;
    }
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

// joins the parts of a token (rising order) and adds the sink: a block per (token, head), a thread per dim
template <typename T>
__global__ __launch_bounds__(128) void attn_mixed_join_kernel(T* __restrict__ out, AttnMixed a, int hd) {
    const int token = blockIdx.x, h = blockIdx.y, nh = a.nh;
    const float* pm = a.part_ml + (size_t)token * a.n_parts * nh * 2;
    const float sk = a.sink ? a.sink[h] : -INFINITY;
    float top = sk;
    for (int part = 0; part < a.n_parts; ++part)
        if (pm[(part * nh + h) * 2 + 1] > 0.f) top = fmaxf(top, pm[(part * nh + h) * 2]);
    for (int d = threadIdx.x; d < hd; d += 128) {
        float den = a.sink ? expf(sk - top) : 0.f, num = 0.f;
        for (int part = 0; part < a.n_parts; ++part) {
            const float m = pm[(part * nh + h) * 2], l = pm[(part * nh + h) * 2 + 1];
            if (!(l > 0.f)) continue;                                         // a part without keys: what it holds is not read
            const float f = expf(m - top);
            den = fmaf(l, f, den);
            num = fmaf(a.part_acc[(((size_t)token * a.n_parts + part) * nh + h) * hd + d], f, num);
        }
        out[((size_t)token * nh + h) * hd + d] = from_f32<T>(den > 0.f ? num / den : 0.f);
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
                             int page_size, int n_pages, float scale, int window, int keep_first, int chunk, const float* slopes,
                             const float* talk, const float* sink, int part_keys, int n_parts, float* part_acc, float* part_ml,
                             hipStream_t stream) {
    FL_CHECK(n >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attn_mixed: bad head counts %d/%d", nh, nkv);
    FL_CHECK(hd > 0 && hd % 8 == 0, "attn_mixed: heads are stored in multiples of 8 values, got %d", hd);
    FL_CHECK(window >= 0 && keep_first >= 0 && chunk >= 0 && !(window > 0 && chunk > 0), "attn_mixed: a window of %d keys, %d kept first tokens, chunks of %d", window, keep_first, chunk);
    FL_CHECK(nh <= fl_attn_mixed_max_heads(hd), "attn_mixed: %d heads of %d values are more than a block holds (%d)", nh, hd,
             fl_attn_mixed_max_heads(hd));
    FL_CHECK(part_keys >= 0 && part_keys % AM_CHUNK == 0, "attn_mixed: parts of %d keys (a multiple of %d wanted)", part_keys, AM_CHUNK);
    FL_CHECK(part_keys == 0 || (n_parts > 0 && n_parts <= 65535 && part_acc && part_ml), "attn_mixed: parts without their buffers");
    if (n == 0) return 0;
    PagedCache c{(void*)cache_base, nkv, page_size, hd, n_pages};
    AttnMixed a{positions, tok_seq, block_table, max_blocks, nh, scale, window, keep_first, chunk, slopes, talk, sink,
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
        if (dtype == FL_F32) attn_mixed_join_kernel<float><<<dim3(n, nh), 128, 0, stream>>>((float*)out, a, hd);
        else attn_mixed_join_kernel<bf16_t><<<dim3(n, nh), 128, 0, stream>>>((bf16_t*)out, a, hd);
        FL_LAUNCH_CHECK();
    }
#undef FL_AM_T
#undef FL_AM
    return 0;
}
FL_RECORDABLE(fl_attn_mixed)


// ---------------------------------------------------------------------------------------------------------
// The same attention on the matrix cores, for bfloat16 caches: a block of eight waves takes up to 16
// consecutive query tokens of one request with ALL heads and walks their keys in chunks of 32 (aligned to
// absolute positions).  Per chunk, with a barrier between the phases:
//   1. raw[g][query][key] = scale * Q_g . K^T - slope_g * (i - j)      v_mfma_f32_16x16x32_bf16, float into LDS;
//      the (head, half chunk) tiles are dealt out to the waves, operands come straight from q and the pages
//   2. score[h][pair] = sum_g talk[h][g] * raw[g][pair]                v_mfma_f32_16x16x4_f32 (true 32-bit): the
//      mixing matrix is the A operand, 16 (query, key) pairs are a B operand's columns, both read from LDS
//      (left out, with its barrier, where there is no mixing matrix: phase 1 then writes the scores where phase 3 reads)
//   3. a thread per (head, query) row: mask, running maximum and sum (they stay in that thread's registers from
//      chunk to chunk), weights as bfloat16 into LDS, and the factor by which the row's output shrinks
//   4. out[h][query][:] = factor * out + P_h . V                        v_mfma_f32_16x16x32_bf16; a wave owns up to four
//      consecutive heads in phases 1 and 4, and heads that share a key/value head share the operands read from the
//      pages; values lie transposed in a page, so eight keys of one dim are one 16-byte load
// Which block takes which tile is found from the step's own lists (first row and rows of every request).
// With part_keys > 0 a tile's keys are dealt out to n_parts blocks as above and joined by the same kernel.
#define AT_ROWS 16
#define AT_CHUNK 32
#define AT_THREADS 512
#define AT_WAVES 8
#define AT_RAW_Q (AT_CHUNK + 4)                 // floats per query row of raw: the four row groups of a score tile fall on two bank halves
#define AT_RAW_LD (AT_ROWS * AT_RAW_Q + 16)     // floats per head of raw (the 16 spread the four heads of an operand over the banks)
#define AT_SC_LD (AT_ROWS * (AT_CHUNK + 1) + 4) // floats per head of score: rows of 33 (a thread walks a row), heads four apart on two bank halves
#define AT_P_LD 40                              // bfloat16 per row of weights
#define AT_MAX_HEADS 32

struct AttnTiles {
    const int* seq_q_start; const int* seq_q_len; int n_seqs;
};

template <int DT>
__global__ __launch_bounds__(AT_THREADS) void attn_mixed_tiled_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                                                                       PagedCache cache, AttnMixed a, AttnTiles tl) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ int s_tile[4];
    const int nh = a.nh, hd = cache.head_dim, ps = cache.page_size;
    const int HP = (nh + 15) & ~15;
    float* raw = lds;                                   // [HP][AT_RAW_LD]
    float* sc = raw + HP * AT_RAW_LD;                   // [HP][16][33]
    float* corr = sc + HP * AT_SC_LD;                   // [HP][16]
    float* tk = corr + HP * AT_ROWS;                    // [HP][HP + 1]
    bf16_t* pb = (bf16_t*)raw;                          // [nh][16][AT_P_LD]: the weights take raw's place once it is mixed
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;

    // ---- which rows: tile blockIdx.x of the requests' portions, 16 rows each (the requests' row counts are fetched by
    // all threads at once, then one thread walks them in LDS)
    int* s_len = (int*)lds;
    for (int s0 = 0, t = blockIdx.x, done = 0; s0 < tl.n_seqs && !done; s0 += AT_THREADS) {
        const int ns = min(AT_THREADS, tl.n_seqs - s0);
        if (tid < ns) s_len[tid] = tl.seq_q_len[s0 + tid];
        if (tid == 0) s_tile[0] = -1;
        __syncthreads();
        if (tid == 0) {
            for (int s = 0; s < ns; ++s) {
                const int len = s_len[s], nt = (len + AT_ROWS - 1) / AT_ROWS;
                if (t < nt) {
                    s_tile[0] = s0 + s; s_tile[1] = tl.seq_q_start[s0 + s] + AT_ROWS * t; s_tile[2] = min(AT_ROWS, len - AT_ROWS * t);
                    break;
                }
                t -= nt;
            }
            s_tile[3] = t;
        }
        __syncthreads();
        done = s_tile[0] >= 0;
        t = s_tile[3];
        __syncthreads();
    }
    if (tl.n_seqs <= 0) return;
    const int seq = s_tile[0], row0 = s_tile[1], cnt = s_tile[2];
    if (seq < 0) return;
    const int p_first = a.positions[row0], p_last = p_first + cnt - 1;
    const int* table = a.block_table + (size_t)seq * a.max_blocks;
    const int safe_page = table[p_last / ps];
    const bool live = safe_page >= 0 && safe_page < cache.n_pages;      // (a padding row of a fixed-size batch has no page)
    const int lo = am_mask_lo(a, p_first);             // (the first key of a row's window or chunk never falls as the rows go on)
    const int kept = min(a.keep_first, lo);            // the keys [0, kept) are seen beside the rows' own runs; the first part's block takes them
    int k0 = lo, k1 = p_last;
    if (a.part_keys > 0) {
        const int part = lo / a.part_keys + blockIdx.y;
        k0 = max(lo, part * a.part_keys);
        k1 = min(p_last, (part + 1) * a.part_keys - 1);
    }
    if (!live || k0 > k1) {
        if (a.part_keys > 0) {
            for (int e = tid; e < cnt * nh; e += AT_THREADS) {
                float* pm = a.part_ml + (((size_t)(row0 + e / nh) * a.n_parts + blockIdx.y) * nh + e % nh) * 2;
                pm[0] = -INFINITY; pm[1] = 0.f;
            }
        } else {
            for (int e = tid; e < cnt * nh * hd; e += AT_THREADS) out[(size_t)row0 * nh * hd + e] = (bf16_t)0.f;
        }
        return;
    }
    const int group = nh / cache.n_kv_heads;
    const bool mixes = a.talk != nullptr;              // (the same for every block: a mixing matrix, or every head for itself)
    const bf16_t* kv = (const bf16_t*)cache.base;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // ---- the mixing matrix (the unit matrix without one), zeros around it up to a multiple of 16: A operands are read from here
    for (int e = tid; e < HP * HP; e += AT_THREADS) {
        const int h = e / HP, g = e % HP;
        tk[h * (HP + 1) + g] = (h < nh && g < nh) ? (a.talk ? a.talk[h * nh + g] : (h == g ? 1.f : 0.f)) : 0.f;
    }
    for (int e = tid; e < (HP - nh) * AT_RAW_LD; e += AT_THREADS) raw[nh * AT_RAW_LD + e] = 0.f;     // heads that do not exist
    // ---- the row (head, query) this thread keeps the softmax of
    const int rh = tid >> 4, rq = tid & 15;
    const bool row_on = rh < nh && rq < cnt;
    const int rp = p_first + rq;
    const int own_lo = am_mask_lo(a, rp);              // this row sees j in [own_lo, rp] and j < keep_first
    float rm = -INFINITY, rl = 0.f;
    // keys that every row of the tile sees: from the last row's first key to the first row's position, inside this block's part
    const int all_lo = max(k0, am_mask_lo(a, p_last)), all_hi = min(k1, p_first);
    const int main_k0 = k0, main_k1 = k1;
    f32x4 o[4][DT];
#pragma unroll
    for (int hi = 0; hi < 4; ++hi)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[hi][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    constexpr int KS = (DT + 1) / 2;                     // steps of 32 dims in a score product
    const int HPW = (nh + AT_WAVES - 1) / AT_WAVES;      // heads per wave, consecutive ones: at most 4
    __syncthreads();

    for (int range = 0; range < 2; ++range) {
    // two runs of keys: the kept first tokens (if the mask hides what follows them), then the rows' own
    if (range == 0) {
        if (kept <= 0 || (a.part_keys > 0 && blockIdx.y != 0)) continue;
        k0 = 0; k1 = kept - 1;
    } else {
        k0 = main_k0; k1 = main_k1;
    }
    const int r_hi = min(k1, rp);
    auto seen = [&](int j) { return j >= k0 && j <= r_hi && (j >= own_lo || j < a.keep_first); };
    for (int base = (k0 / AT_CHUNK) * AT_CHUNK; base <= k1; base += AT_CHUNK) {
        // ---- 1. raw scores: a wave takes HPW consecutive heads
        {
            const size_t head_stride = (size_t)ps * hd;
            const bf16_t* kpage[2];
            int jpos[2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                jpos[kt] = base + 16 * kt + li;
                int page = jpos[kt] <= p_last ? table[jpos[kt] / ps] : safe_page;
                if (page < 0 || page >= cache.n_pages) page = safe_page;
                kpage[kt] = kv + cache_k_offset(cache, page, 0, jpos[kt] % ps, 0);
            }
            // the keys of a key/value head are loaded once for the heads that share it (they follow one another in a
            // wave)
            auto load_q = [&](int g, bf16x8* qf) {
                const bf16_t* qrow = q + ((size_t)(row0 + li) * nh + g) * hd;
#pragma unroll
                for (int s = 0; s < KS; ++s) {
                    const int d = 32 * s + 8 * lg;
                    qf[s] = (d < hd && li < cnt && g < nh) ? *(const bf16x8*)(qrow + d) : zero8;
                }
            };
            bf16x8 kf[2][KS], qf[KS];
            int kvh_held = -1;
#pragma unroll
            for (int hi = 0; hi < 4; ++hi) {
                const int g = wave * HPW + hi;
                if (hi >= HPW || g >= nh) continue;
                const int kvh = g / group;
                if (kvh != kvh_held) {
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int s = 0; s < KS; ++s) {
                            const int d = 32 * s + 8 * lg;
                            kf[kt][s] = d < hd ? *(const bf16x8*)(kpage[kt] + kvh * head_stride + d) : zero8;
                        }
                    kvh_held = kvh;
                }
                load_q(g, qf);
                const float slope = a.slopes ? a.slopes[g] : 0.f;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < KS; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[s], kf[kt][s], acc, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int qq = 4 * lg + r;
                        const float sv = acc[r] * a.scale - slope * (float)(p_first + qq - jpos[kt]);
                        // (without a mixing matrix a head's score is its own raw score: it goes where phase 3 reads, and phase 2 is left out)
                        if (mixes) raw[g * AT_RAW_LD + qq * AT_RAW_Q + 16 * kt + li] = sv;
                        else sc[g * AT_SC_LD + qq * (AT_CHUNK + 1) + 16 * kt + li] = sv;
                    }
                }
            }
        }
        __syncthreads();
        // ---- 2. the heads' scores mixed: 16 pairs at a time, pairs of the queries that exist
        if (mixes) {
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            if (16 * hb >= HP) continue;
            for (int pt = wave; pt < 2 * cnt; pt += AT_WAVES) {
                f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < AT_MAX_HEADS / 4; ++kk) {
                    if (4 * kk >= HP) continue;
                    c = __builtin_amdgcn_mfma_f32_16x16x4f32(tk[(16 * hb + li) * (HP + 1) + 4 * kk + lg], raw[(4 * kk + lg) * AT_RAW_LD + (pt >> 1) * AT_RAW_Q + 16 * (pt & 1) + li], c, 0, 0, 0);
                }
                const int pair = 16 * pt + li;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    sc[(16 * hb + 4 * lg + r) * AT_SC_LD + (pair >> 5) * (AT_CHUNK + 1) + (pair & 31)] = c[r];
            }
        }
        __syncthreads();
        }
        // ---- 3. the rows' softmax.  Most chunks lie inside every row's window: there no key is tested
        if (rh < nh) {
            u32x4* prow4 = (u32x4*)(pb + (rh * AT_ROWS + rq) * AT_P_LD);      // eight weights a store
            const float* srow = sc + rh * AT_SC_LD + rq * (AT_CHUNK + 1);
            const bool inside = range == 1 && base >= all_lo && base + AT_CHUNK - 1 <= all_hi;     // (the same for the whole block)
            auto pack = [](float e0, float e1) {
                const bf16_t b0 = (bf16_t)e0, b1 = (bf16_t)e1;
                return (unsigned)__builtin_bit_cast(unsigned short, b0) | ((unsigned)__builtin_bit_cast(unsigned short, b1) << 16);
            };
            if (inside && row_on) {
                float sv[AT_CHUNK];
#pragma unroll
                for (int j = 0; j < AT_CHUNK; ++j) sv[j] = srow[j];
                float mx = sv[0];
#pragma unroll
                for (int j = 1; j < AT_CHUNK; ++j) mx = fmaxf(mx, sv[j]);
                const float m_new = fmaxf(rm, mx);
                const float cr = rm == -INFINITY ? 0.f : __expf(rm - m_new);
                float sum = 0.f;
#pragma unroll
                for (int j8 = 0; j8 < AT_CHUNK; j8 += 8) {
                    u32x4 w;
#pragma unroll
                    for (int j = 0; j < 8; j += 2) {
                        const float e0 = __expf(sv[j8 + j] - m_new), e1 = __expf(sv[j8 + j + 1] - m_new);
                        sum += e0 + e1;
                        w[j >> 1] = pack(e0, e1);
                    }
                    prow4[j8 >> 3] = w;
                }
                rl = rl * cr + sum;
                rm = m_new;
                corr[rh * AT_ROWS + rq] = cr;
            } else {
                float mx = -INFINITY;
                if (row_on)
                    for (int j = 0; j < AT_CHUNK; ++j)
                        if (seen(base + j)) mx = fmaxf(mx, srow[j]);
                if (mx == -INFINITY) {                                        // no key of this chunk for this row
                    for (int j8 = 0; j8 < AT_CHUNK / 8; ++j8) prow4[j8] = (u32x4){0u, 0u, 0u, 0u};
                    corr[rh * AT_ROWS + rq] = 1.f;
                } else {
                    const float m_new = fmaxf(rm, mx);
                    const float cr = rm == -INFINITY ? 0.f : __expf(rm - m_new);
                    float sum = 0.f;
                    for (int j8 = 0; j8 < AT_CHUNK; j8 += 8) {
                        u32x4 w;
#pragma unroll
                        for (int j = 0; j < 8; j += 2) {
                            const int jp = base + j8 + j;
                            const float e0 = seen(jp) ? __expf(srow[j8 + j] - m_new) : 0.f;
                            const float e1 = seen(jp + 1) ? __expf(srow[j8 + j + 1] - m_new) : 0.f;
                            sum += e0 + e1;
                            w[j >> 1] = pack(e0, e1);
                        }
                        prow4[j8 >> 3] = w;
                    }
                    rl = rl * cr + sum;
                    rm = m_new;
                    corr[rh * AT_ROWS + rq] = cr;
                }
            }
        }
        __syncthreads();
        // ---- 4. the weighted sums of the values
        {
            const int jr = base + 8 * lg;                                      // this lane's run of eight keys
            int page = jr <= p_last ? table[jr / ps] : -1;
            const bool run_on = page >= 0 && page < cache.n_pages && jr <= k1;
            if (!run_on) page = safe_page;
            const bf16_t* vpage = kv + cache_v_offset(cache, page, 0, jr % ps, 0);
            const size_t head_stride = (size_t)ps * hd;
            constexpr int DH = DT / 2;                                         // the value dims in two halves: fewer operands held at a time
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                bf16x8 vf[DH];
                int kvh_held = -1;
#pragma unroll
                for (int hi = 0; hi < 4; ++hi) {
                    const int h = wave * HPW + hi;
                    if (hi >= HPW || h >= nh) continue;
                    const int kvh = h / group;
                    if (kvh != kvh_held) {
                        const bf16_t* vbase = vpage + kvh * head_stride;
#pragma unroll
                        for (int dt = 0; dt < DH; ++dt) {
                            const int d = 16 * (half * DH + dt) + li;
                            vf[dt] = (run_on && d < hd) ? *(const bf16x8*)(vbase + (size_t)d * ps) : zero8;
                        }
                        if (jr + 7 > k1) {                                     // keys that nobody wrote yet may hold anything
#pragma unroll
                            for (int dt = 0; dt < DH; ++dt)
#pragma unroll
                                for (int e = 0; e < 8; ++e)
                                    if (jr + e > k1) vf[dt][e] = (bf16_t)0.f;
                        }
                        kvh_held = kvh;
                    }
                    float cr[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) cr[r] = corr[h * AT_ROWS + 4 * lg + r];
                    const bf16x8 pf = *(const bf16x8*)(pb + (h * AT_ROWS + li) * AT_P_LD + 8 * lg);
#pragma unroll
                    for (int dt = 0; dt < DH; ++dt) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[hi][half * DH + dt][r] *= cr[r];
                        o[hi][half * DH + dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf[dt], o[hi][half * DH + dt], 0, 0, 0);
                    }
                }
            }
        }
        __syncthreads();
    }
    }

    // ---- the rows' maxima and sums go to the waves that hold the outputs (or to the parts' scratch)
    float* hm = sc;
    float* hl = sc + HP * AT_ROWS;
    if (rh < nh) {
        hm[rh * AT_ROWS + rq] = rm;
        hl[rh * AT_ROWS + rq] = rl;
        if (a.part_keys > 0 && rq < cnt) {
            float* pm = a.part_ml + (((size_t)(row0 + rq) * a.n_parts + blockIdx.y) * nh + rh) * 2;
            pm[0] = rm; pm[1] = rl;
        }
    }
    __syncthreads();
#pragma unroll
    for (int hi = 0; hi < 4; ++hi) {
        const int h = wave * HPW + hi;
        if (hi >= HPW || h >= nh) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int qq = 4 * lg + r;
            if (qq >= cnt) continue;
            float f = 1.f;
            if (a.part_keys == 0) {
                const float m = hm[h * AT_ROWS + qq], l = hl[h * AT_ROWS + qq];
                const float sk = a.sink ? a.sink[h] : -INFINITY;
                const float top = fmaxf(m, sk);
                const float fm = expf(m - top);
                const float den = l * fm + (a.sink ? expf(sk - top) : 0.f);
                f = den > 0.f ? fm / den : 0.f;
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = 16 * dt + li;
                if (d >= hd) continue;
                if (a.part_keys > 0) a.part_acc[(((size_t)(row0 + qq) * a.n_parts + blockIdx.y) * nh + h) * hd + d] = o[hi][dt][r];
                else out[((size_t)(row0 + qq) * nh + h) * hd + d] = (bf16_t)(o[hi][dt][r] * f);
            }
        }
    }
}

extern "C" int fl_attn_mixed_tiled_fits(int nh, int hd, int page_size) {
    return nh >= 1 && nh <= AT_MAX_HEADS && hd % 8 == 0 && hd <= 128 && page_size % 8 == 0;
}

// ``n_tiles``: the sum over the step's requests of ceil(rows / 16), which the caller knows from the rows per request
extern "C" int fl_attn_mixed_tiled(const void* q, void* out, const void* cache_base, const int* positions, const int* block_table,
                                   int max_blocks, const int* seq_q_start, const int* seq_q_len, int n_seqs, int n_tiles, int n,
                                   int nh, int nkv, int hd, int page_size, int n_pages, float scale, int window, int keep_first, int chunk,
                                   const float* slopes, const float* talk, const float* sink, int part_keys, int n_parts, float* part_acc,
                                   float* part_ml, hipStream_t stream) {
    FL_CHECK(n >= 0 && nkv > 0 && nh % nkv == 0, "attn_mixed_tiled: bad head counts %d/%d", nh, nkv);
    FL_CHECK(fl_attn_mixed_tiled_fits(nh, hd, page_size), "attn_mixed_tiled: %d heads of %d values over pages of %d are not what the kernel takes",
             nh, hd, page_size);
    FL_CHECK(window >= 0 && n_seqs >= 0 && n_tiles >= 0 && n_tiles <= n, "attn_mixed_tiled: bad window or tile count");
    FL_CHECK(keep_first >= 0 && chunk >= 0 && !(window > 0 && chunk > 0), "attn_mixed_tiled: a window of %d keys, %d kept first tokens, chunks of %d", window, keep_first, chunk);
    FL_CHECK(part_keys >= 0 && part_keys % AT_CHUNK == 0, "attn_mixed_tiled: parts of %d keys (a multiple of %d wanted)", part_keys, AT_CHUNK);
    FL_CHECK(part_keys == 0 || (n_parts > 0 && n_parts <= 65535 && part_acc && part_ml), "attn_mixed_tiled: parts without their buffers");
    if (n == 0 || n_tiles == 0) return 0;
    PagedCache c{(void*)cache_base, nkv, page_size, hd, n_pages};
    AttnMixed a{positions, nullptr, block_table, max_blocks, nh, scale, window, keep_first, chunk, slopes, talk, sink,
                part_keys, part_keys ? n_parts : 1, part_acc, part_ml};
    AttnTiles tl{seq_q_start, seq_q_len, n_seqs};
    const int HP = (nh + 15) & ~15;
    const size_t lds = 4 * ((size_t)HP * AT_RAW_LD + (size_t)HP * AT_SC_LD + (size_t)HP * AT_ROWS + (size_t)HP * (HP + 1));
    dim3 grid(n_tiles, a.n_parts);
#define FL_AT(DT)                                                                                                        \
    do {                                                                                                                 \
        static bool configured = false;                                                                                  \
        if (!configured) {                                                                                               \
            const hipError_t e = hipFuncSetAttribute((const void*)attn_mixed_tiled_kernel<DT>,                           \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);            \
            FL_CHECK(e == hipSuccess, "attn_mixed_tiled: hipFuncSetAttribute failed: %s", hipGetErrorString(e));         \
            configured = true;                                                                                           \
        }                                                                                                                \
        attn_mixed_tiled_kernel<DT><<<grid, AT_THREADS, lds, stream>>>((const bf16_t*)q, (bf16_t*)out, c, a, tl);        \
    } while (0)
    if (hd <= 32) FL_AT(2);
    else if (hd <= 64) FL_AT(4);
    else FL_AT(8);
#undef FL_AT
    FL_LAUNCH_CHECK();
    if (part_keys > 0) {
        attn_mixed_join_kernel<bf16_t><<<dim3(n, nh), 128, 0, stream>>>((bf16_t*)out, a, hd);
        FL_LAUNCH_CHECK();
    }
    return 0;
}
FL_RECORDABLE(fl_attn_mixed_tiled)
