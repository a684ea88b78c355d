// Layer norm with gain and bias, and what a decoder that norms its sublayers' OUTPUTS needs around it.
//
//   fl_layernorm       out = (v - mean) / sqrt(var + eps) * w + b of v = x (+ delta), var = mean((v - mean)^2);
//                      resid_out and rows as for fl_rmsnorm; out may be x itself (float, no rows)
//   fl_layernorm_add   resid += layernorm(delta); optionally the new stream once more in the compute type,
//                      for the sublayer that reads the stream itself next
//   fl_embed_positions out[t] = table[token[t]] + pos_table[position[t]] (a learned row per position, not scaled)
//   fl_cast_rows       a float matrix in the compute type
//   fl_scale_inplace   x *= s
// All sums are float; mean and variance are two passes (sum, then sum of squared deviations), each thread
// adding its values in rising order and the block's partial sums in a fixed tree: a row's result does not
// depend on what else the step holds.  In a step of few rows (where a pass over a row is a wait for memory and
// little else), rows of up to 8,192 values whose length is a multiple of four are read once, 16 bytes at a time, and
// stay in registers through both passes and the output; otherwise a row is read thrice.
#include "common.h"
#include "api.h"
#include "recordable.h"

// one value's result, written with the fused multiply-add spelt out so that every path rounds alike
__device__ __forceinline__ float layernorm_value(float v, float mean, float inv, float w, float b) {
    return fmaf((v - mean) * inv, w, b);
}

template <typename F>
__device__ __forceinline__ void layernorm_row(F&& value, int H, float eps, float* lds, float& mean, float& inv) {
    float s = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) s += value(i);
    mean = block_sum<4>(s, lds) / (float)H;
    float v = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        const float d = value(i) - mean;
        v = fmaf(d, d, v);
    }
    inv = 1.0f / sqrtf(block_sum<4>(v, lds + 4) / (float)H + eps);
}

// the same sums in the same order as layernorm_row_held below, for rows that are not held (every pass reads the row):
// a row's bits do not depend on which of the two ran
__device__ __forceinline__ void layernorm_row4(const float* xr, const float* dr, int H, float eps, float* lds, float& mean, float& inv) {
    const int H4 = H >> 2;
    float s = 0.f;
    for (int i4 = threadIdx.x; i4 < H4; i4 += 256) {
        f32x4 v = *(const f32x4*)(xr + 4 * i4);
        if (dr) v += *(const f32x4*)(dr + 4 * i4);
        s += (v[0] + v[1]) + (v[2] + v[3]);
    }
    mean = block_sum<4>(s, lds) / (float)H;
    float q = 0.f;
    for (int i4 = threadIdx.x; i4 < H4; i4 += 256) {
        f32x4 v = *(const f32x4*)(xr + 4 * i4);
        if (dr) v += *(const f32x4*)(dr + 4 * i4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float d = v[e] - mean;
            q = fmaf(d, d, q);
        }
    }
    inv = 1.0f / sqrtf(block_sum<4>(q, lds + 4) / (float)H + eps);
}

#define LN_HELD 8            // groups of four values a thread holds

// the row in registers: v[k] = values 4 (tid + 256 k) .. + 3 of x (+ delta); mean and 1 / sqrt(var + eps) of it
__device__ __forceinline__ void layernorm_row_held(const float* xr, const float* dr, int H, float eps, float* lds, f32x4* v,
                                                   float& mean, float& inv) {
    const int H4 = H >> 2;
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < LN_HELD; ++k) {
        const int i4 = threadIdx.x + 256 * k;
        v[k] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (i4 < H4) {
            v[k] = *(const f32x4*)(xr + 4 * i4);
            if (dr) v[k] += *(const f32x4*)(dr + 4 * i4);
            s += (v[k][0] + v[k][1]) + (v[k][2] + v[k][3]);
        }
    }
    mean = block_sum<4>(s, lds) / (float)H;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < LN_HELD; ++k) {
        if (threadIdx.x + 256 * k < H4) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float d = v[k][e] - mean;
                q = fmaf(d, d, q);
            }
        }
    }
    inv = 1.0f / sqrtf(block_sum<4>(q, lds + 4) / (float)H + eps);
}

#define LN_FEW_ROWS 256
static inline bool layernorm_holds(int n, int H) { return n <= LN_FEW_ROWS && (H & 3) == 0 && H <= 4 * 256 * LN_HELD; }

template <typename T> __device__ __forceinline__ void store4(T* p, f32x4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, f32x4 v) { *(f32x4*)p = v; }
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4 v) {
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *(bf16x4*)p = o;
}

template <typename TOut>
__global__ __launch_bounds__(256) void layernorm_kernel(const float* x, const float* __restrict__ delta,
                                                        float* resid_out, const int* __restrict__ rows,
                                                        const float* __restrict__ w, const float* __restrict__ b, TOut* out,
                                                        int H, float eps, bool held) {
    __shared__ float lds[8];
    const size_t src = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
    const float* xr = x + src * H;
    const float* dr = delta ? delta + src * H : nullptr;
    TOut* o = out + (size_t)blockIdx.x * H;
    float mean, inv;
    if (held) {
        f32x4 v[LN_HELD];
        layernorm_row_held(xr, dr, H, eps, lds, v, mean, inv);
#pragma unroll
        for (int k = 0; k < LN_HELD; ++k) {
            const int i = 4 * (threadIdx.x + 256 * k);
            if (i >= H) continue;
            if (resid_out) *(f32x4*)(resid_out + src * H + i) = v[k];
            const f32x4 w4 = *(const f32x4*)(w + i), b4 = b ? *(const f32x4*)(b + i) : (f32x4){0.f, 0.f, 0.f, 0.f};
            f32x4 y;
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = layernorm_value(v[k][e], mean, inv, w4[e], b4[e]);
            store4<TOut>(o + i, y);
        }
        return;
    }
    auto value = [&](int i) { return dr ? xr[i] + dr[i] : xr[i]; };
    if ((H & 3) == 0) layernorm_row4(xr, dr, H, eps, lds, mean, inv);
    else layernorm_row(value, H, eps, lds, mean, inv);
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = value(i);
        if (resid_out) resid_out[src * H + i] = v;
        o[i] = from_f32<TOut>(layernorm_value(v, mean, inv, w[i], b ? b[i] : 0.f));
    }
}

extern "C" int fl_layernorm(const float* x, const float* delta, float* resid_out, const int* rows, const float* w,
                            const float* b, void* out, int out_dtype, int n, int H, float eps, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && x && w && out, "layernorm: bad sizes or a missing tensor");
    FL_CHECK(!(resid_out && rows), "layernorm: the sum is not stored back for picked rows");
    if (n == 0) return 0;
    if (out_dtype == FL_F32) layernorm_kernel<float><<<n, 256, 0, stream>>>(x, delta, resid_out, rows, w, b, (float*)out, H, eps, layernorm_holds(n, H));
    else if (out_dtype == FL_BF16) layernorm_kernel<bf16_t><<<n, 256, 0, stream>>>(x, delta, resid_out, rows, w, b, (bf16_t*)out, H, eps, layernorm_holds(n, H));
    else FL_CHECK(false, "layernorm: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_layernorm)

template <typename TC>
__global__ __launch_bounds__(256) void layernorm_add_kernel(const float* __restrict__ delta, const float* __restrict__ w,
                                                            const float* __restrict__ b, float* __restrict__ resid,
                                                            TC* __restrict__ cast, int H, float eps, bool held) {
    __shared__ float lds[8];
    const float* dr = delta + (size_t)blockIdx.x * H;
    float* r = resid + (size_t)blockIdx.x * H;
    float mean, inv;
    if (held) {
        f32x4 v[LN_HELD];
        layernorm_row_held(dr, nullptr, H, eps, lds, v, mean, inv);
#pragma unroll
        for (int k = 0; k < LN_HELD; ++k) {
            const int i = 4 * (threadIdx.x + 256 * k);
            if (i >= H) continue;
            const f32x4 w4 = *(const f32x4*)(w + i), b4 = b ? *(const f32x4*)(b + i) : (f32x4){0.f, 0.f, 0.f, 0.f};
            f32x4 y = *(const f32x4*)(r + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] += layernorm_value(v[k][e], mean, inv, w4[e], b4[e]);
            *(f32x4*)(r + i) = y;
            if (cast) store4<TC>(cast + (size_t)blockIdx.x * H + i, y);
        }
        return;
    }
    auto value = [&](int i) { return dr[i]; };
    if ((H & 3) == 0) layernorm_row4(dr, nullptr, H, eps, lds, mean, inv);
    else layernorm_row(value, H, eps, lds, mean, inv);
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = r[i] + layernorm_value(dr[i], mean, inv, w[i], b ? b[i] : 0.f);
        r[i] = v;
        if (cast) cast[(size_t)blockIdx.x * H + i] = from_f32<TC>(v);
    }
}

extern "C" int fl_layernorm_add(const float* delta, const float* w, const float* b, float* resid, void* cast, int cast_dtype,
                                int n, int H, float eps, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && delta && w && resid, "layernorm_add: bad sizes or a missing tensor");
    if (n == 0) return 0;
    if (!cast || cast_dtype == FL_F32) layernorm_add_kernel<float><<<n, 256, 0, stream>>>(delta, w, b, resid, (float*)cast, H, eps, layernorm_holds(n, H));
    else if (cast_dtype == FL_BF16) layernorm_add_kernel<bf16_t><<<n, 256, 0, stream>>>(delta, w, b, resid, (bf16_t*)cast, H, eps, layernorm_holds(n, H));
    else FL_CHECK(false, "layernorm_add: unknown dtype %d", cast_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_layernorm_add)

template <typename T>
__global__ __launch_bounds__(256) void embed_positions_kernel(const T* __restrict__ table, const T* __restrict__ pos_table,
                                                              const int* __restrict__ tokens, const int* __restrict__ positions,
                                                              float* __restrict__ out, int H, int V, int P) {
    const int tok = tokens[blockIdx.x], pos = positions[blockIdx.x];
    float* o = out + (size_t)blockIdx.x * H;
    const bool ok = tok >= 0 && tok < V && pos >= 0 && pos < P;        // (padding rows of a fixed-size batch: zeros)
    for (int i = threadIdx.x; i < H; i += 256)
        o[i] = ok ? to_f32(table[(size_t)tok * H + i]) + to_f32(pos_table[(size_t)pos * H + i]) : 0.f;
}

extern "C" int fl_embed_positions(const void* table, const void* pos_table, int dtype, const int* tokens, const int* positions,
                                  float* out, int n, int H, int V, int P, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && V > 0 && P > 0, "embed_positions: bad sizes");
    if (n == 0) return 0;
    if (dtype == FL_F32)
        embed_positions_kernel<float><<<n, 256, 0, stream>>>((const float*)table, (const float*)pos_table, tokens, positions, out, H, V, P);
    else if (dtype == FL_BF16)
        embed_positions_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)table, (const bf16_t*)pos_table, tokens, positions, out, H, V, P);
    else FL_CHECK(false, "embed_positions: unknown dtype %d", dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_embed_positions)

template <typename T>
__global__ __launch_bounds__(256) void cast_rows_kernel(const float* __restrict__ x, T* __restrict__ out, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) out[i] = from_f32<T>(x[i]);
}

extern "C" int fl_cast_rows(const float* x, void* out, int out_dtype, long total, hipStream_t stream) {
    FL_CHECK(total >= 0, "cast_rows: bad size");
    if (total == 0) return 0;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (out_dtype == FL_F32) cast_rows_kernel<float><<<blocks, 256, 0, stream>>>(x, (float*)out, total);
    else if (out_dtype == FL_BF16) cast_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (bf16_t*)out, total);
    else FL_CHECK(false, "cast_rows: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_cast_rows)

__global__ __launch_bounds__(256) void scale_inplace_kernel(float* __restrict__ x, long total, float s) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < total) x[i] *= s;
}

extern "C" int fl_scale_inplace(float* x, long total, float s, hipStream_t stream) {
    FL_CHECK(total >= 0, "scale_inplace: bad size");
    if (total == 0) return 0;
    scale_inplace_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(x, total, s);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_scale_inplace)
