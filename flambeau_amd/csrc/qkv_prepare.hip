// What stands between the joined q/k/v projection of a softmax-attention mixer and attention itself,
// for mixers whose queries and keys are normed and whose heads differ in key and value size:
//   * a norm over the WHOLE projection of q (and of k) with a gain per value, before rotation
//     (x / sqrt(mean(x^2) + eps) * w over all heads at once), or none;
//   * rotation of the first `rot` dims of every head from the step's table of cosines and sines, pairs
//     (i, i + rot/2) ("half") or (2i, 2i + 1) ("interleaved");
//   * every head of q and k divided by its root mean square after rotation, with no gain or with a gain per
//     head dim that all heads of q (of k) share, or not;
//   * values blended with those an earlier layer made for the same token,
//     v <- (1 - lambda) v + lambda v_first, or kept as that first layer's for later ones;
//   * q stored for the attention kernels, k and v stored into the paged cache at the token's position;
//   * ahead of all of it, the projections' biases (one value per column of the joined projection), or none.
// Heads are stored `hdp` wide (hdp >= max(D, Dv)): keys are padded with zeros behind D, values behind
// Dv, queries behind D, so that attention kernels of one head size serve key and value sizes that differ.
// The projection arrives in float; everything here is float, only the stores are in the cache's type.
#include "common.h"
#include "api.h"
#include "recordable.h"

#define QKV_FEW_TOKENS 64     // up to this many tokens a block forms the projection's sums of squares for itself

struct QkvPrepare {
    const float* proj; int ld; int col_q, col_k, col_v;
    const int* positions; const int* tok_seq; const int* block_table; int max_blocks;
    int nh, D, Dv, hdp;
    int rot, interleaved; const float2* cs;
    const float* qnorm_w; const float* knorm_w; int head_norm; float eps;
    const float* q_head_gain; const float* k_head_gain;   // [D] each, or null: the gain behind the heads' own norm
    float* v_first; int vmix_mode; const float* lambda;
    int write_cache;
    float* row_scales;          // [n][2]: 1 / rms of every token's q and k projection, made by a kernel of its own (or null)
    const float* bias;          // [ld] or null: added to the projection's columns as they are read
};

// The norm over the whole projection of q and of k: 1 / sqrt(mean(x^2) + eps) of both for one token per block.
__global__ __launch_bounds__(256) void qkv_row_scales_kernel(QkvPrepare a, int nkv) {
    __shared__ float lds[8];
    const float* row = a.proj + (size_t)blockIdx.x * a.ld;
    auto at = [&](int c) { return a.bias ? row[c] + a.bias[c] : row[c]; };
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < a.nh * a.D; i += 256) sq = fmaf(at(a.col_q + i), at(a.col_q + i), sq);
    if (a.col_k >= 0) for (int i = threadIdx.x; i < nkv * a.D; i += 256) sk = fmaf(at(a.col_k + i), at(a.col_k + i), sk);
    sq = block_sum<4>(sq, lds);
    sk = block_sum<4>(sk, lds + 4);
    if (threadIdx.x == 0) {
        a.row_scales[2 * blockIdx.x] = 1.0f / sqrtf(sq / (float)(a.nh * a.D) + a.eps);
        a.row_scales[2 * blockIdx.x + 1] = 1.0f / sqrtf(sk / (float)(nkv * a.D) + a.eps);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(QkvPrepare a, T* __restrict__ q_out, PagedCache cache) {
    __shared__ float lds[8];
    const int token = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nh = a.nh, nkv = cache.n_kv_heads, D = a.D, Dv = a.Dv, hdp = a.hdp;
    const float* row = a.proj + (size_t)token * a.ld;
    auto at = [&](int c) { return a.bias ? row[c] + a.bias[c] : row[c]; };       // a column of the projection, its bias added
    const bool has_kv = a.col_k >= 0;                 // (a mixer that reads another layer's keys and values projects queries alone)
    float inv_q = 1.f, inv_k = 1.f;
    if (a.qnorm_w && a.row_scales) {
        inv_q = a.row_scales[2 * token];
        inv_k = a.row_scales[2 * token + 1];
    } else if (a.qnorm_w) {
        // (a step of few tokens: every block sums for itself, in the same order as the kernel above, and a launch is saved)
        float sq = 0.f, sk = 0.f;
        for (int i = threadIdx.x; i < nh * D; i += 256) sq = fmaf(at(a.col_q + i), at(a.col_q + i), sq);
        if (has_kv) for (int i = threadIdx.x; i < nkv * D; i += 256) sk = fmaf(at(a.col_k + i), at(a.col_k + i), sk);
        inv_q = 1.0f / sqrtf(block_sum<4>(sq, lds) / (float)(nh * D) + a.eps);
        inv_k = 1.0f / sqrtf(block_sum<4>(sk, lds + 4) / (float)(nkv * D) + a.eps);
    }
    const int pos = a.positions[token];
    int page = -1, prow = 0;
    if (a.write_cache) {
        page = a.block_table[(size_t)a.tok_seq[token] * a.max_blocks + pos / cache.page_size];
        if (page >= cache.n_pages) page = -1;             // (padding rows of a fixed-size batch have no page)
        prow = pos % cache.page_size;
    }
    const int half = a.rot >> 1;
    // q and k heads: a wave per head, a lane per head dim (and the dims 64, 128, ... further); the heads of a token
    // are spread over blocks of four waves (every block forms the projection's sums of squares for itself)
    const int head = blockIdx.y * 4 + wave;
    if (head < nh + (has_kv ? nkv : 0)) {
        const bool is_q = head < nh;
        const int h = is_q ? head : head - nh;
        const int src = (is_q ? a.col_q : a.col_k) + h * D;
        const float* gain = is_q ? a.qnorm_w : a.knorm_w;
        const float inv = is_q ? inv_q : inv_k;
        auto value = [&](int d) { return gain ? at(src + d) * inv * gain[h * D + d] : at(src + d); };
        float r[4];
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + 64 * j;
            r[j] = 0.f;
            if (d >= D) continue;
            float v = value(d);
            if (d < a.rot) {
                int i, partner;
                bool first;
                if (a.interleaved) { i = d >> 1; first = !(d & 1); partner = d ^ 1; }
                else { first = d < half; i = first ? d : d - half; partner = first ? d + half : d - half; }
                const float2 c = a.cs[(size_t)token * half + i];
                const float o = value(partner);
                v = first ? v * c.x - o * c.y : v * c.x + o * c.y;
            }
            r[j] = v;
            ss = fmaf(v, v, ss);
        }
        if (a.head_norm) {
            const float f = 1.0f / sqrtf(wave_sum(ss) / (float)D + a.eps);
            const float* hg = is_q ? a.q_head_gain : a.k_head_gain;
#pragma unroll
            for (int j = 0; j < 4; ++j) r[j] *= (hg && lane + 64 * j < D) ? f * hg[lane + 64 * j] : f;
        }
        if (is_q) {
            T* dst = q_out + ((size_t)token * nh + h) * hdp;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (lane + 64 * j < hdp) dst[lane + 64 * j] = from_f32<T>(r[j]);
        } else if (page >= 0) {
            T* dst = (T*)cache.base + cache_k_offset(cache, page, h, prow, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (lane + 64 * j < hdp) dst[lane + 64 * j] = from_f32<T>(r[j]);
        }
    }
    // v heads: the blocks share their values out
    const float lam = a.vmix_mode == 2 ? a.lambda[0] : 0.f;
    for (int e = blockIdx.y * 256 + threadIdx.x; has_kv && e < nkv * hdp; e += 256 * gridDim.y) {
        const int h = e / hdp, d = e - h * hdp;
        float v = 0.f;
        if (d < Dv) {
            v = at(a.col_v + h * Dv + d);
            const size_t at = (size_t)token * nkv * Dv + h * Dv + d;
            if (a.vmix_mode == 1) a.v_first[at] = v;
            else if (a.vmix_mode == 2) v = (1.0f - lam) * v + lam * a.v_first[at];
        }
        if (page >= 0) ((T*)cache.base)[cache_v_offset(cache, page, h, prow, d)] = from_f32<T>(v);
    }
}

extern "C" int fl_qkv_prepare(const float* proj, int ld, int col_q, int col_k, int col_v, const int* positions,
                              const int* tok_seq, const int* block_table, int max_blocks, void* q_out, void* cache_base,
                              int dtype, int n, int nh, int nkv, int D, int Dv, int hdp, int page_size, int n_pages, int rot,
                              int interleaved, const float* cs, const float* qnorm_w, const float* knorm_w, int head_norm,
                              const float* q_head_gain, const float* k_head_gain, float eps, float* v_first, int vmix_mode, const float* lambda, int write_cache,
                              float* row_scales, const float* bias, hipStream_t stream) {
    FL_CHECK(n >= 0 && nh > 0 && nkv > 0 && D > 0 && Dv > 0 && page_size > 0, "qkv_prepare: bad sizes");
    FL_CHECK(hdp >= D && hdp >= Dv && hdp <= 256, "qkv_prepare: heads of %d and %d values stored %d wide (at most 256)", D, Dv, hdp);
    FL_CHECK(rot >= 0 && rot <= D && rot % 2 == 0, "qkv_prepare: rotated dims %d of head %d", rot, D);
    FL_CHECK(rot == 0 || cs, "qkv_prepare: a rotation needs the step's table of cosines and sines");
    FL_CHECK(ld >= col_q + nh * D && (col_k < 0 || (ld >= col_k + nkv * D && ld >= col_v + nkv * Dv)), "qkv_prepare: columns beyond rows %d wide", ld);
    FL_CHECK(col_k >= 0 || !write_cache, "qkv_prepare: a projection of queries alone writes no cache");
    FL_CHECK(col_k < 0 ? !knorm_w : !qnorm_w == !knorm_w, "qkv_prepare: the norm over the projection needs both gains");
    FL_CHECK(head_norm || (!q_head_gain && !k_head_gain), "qkv_prepare: a gain per head dim without the heads' norm");
    FL_CHECK(vmix_mode >= 0 && vmix_mode <= 2 && (vmix_mode == 0 || v_first) && (vmix_mode != 2 || lambda),
             "qkv_prepare: value blending %d without its buffers", vmix_mode);
    if (n == 0) return 0;
    QkvPrepare a{proj, ld, col_q, col_k, col_v, positions, tok_seq, block_table, max_blocks, nh, D, Dv, hdp,
                 rot, interleaved, (const float2*)cs, qnorm_w, knorm_w, head_norm, eps, q_head_gain, k_head_gain, v_first, vmix_mode, lambda, write_cache,
                 (qnorm_w && n > QKV_FEW_TOKENS) ? row_scales : nullptr, bias};
    PagedCache c{cache_base, nkv, page_size, hdp, n_pages};
    dim3 grid(n, ceil_div(nh + (col_k >= 0 ? nkv : 0), 4));
    FL_CHECK(grid.y <= 65535, "qkv_prepare: %d heads are more than one grid takes", nh + nkv);
    if (a.row_scales) {
        // many tokens: the sums of squares once per token, not once per block of four heads
        qkv_row_scales_kernel<<<n, 256, 0, stream>>>(a, nkv);
        FL_LAUNCH_CHECK();
    }
    if (dtype == FL_F32)
        qkv_prepare_kernel<float><<<grid, 256, 0, stream>>>(a, (float*)q_out, c);
    else if (dtype == FL_BF16)
        qkv_prepare_kernel<bf16_t><<<grid, 256, 0, stream>>>(a, (bf16_t*)q_out, c);
    else
        FL_CHECK(false, "qkv_prepare: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_qkv_prepare)
