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
// depend on what else the step holds.
#include "common.h"
#include "api.h"
#include "recordable.h"

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

template <typename TOut>
__global__ __launch_bounds__(256) void layernorm_kernel(const float* x, const float* __restrict__ delta,
                                                        float* resid_out, const int* __restrict__ rows,
                                                        const float* __restrict__ w, const float* __restrict__ b, TOut* out,
                                                        int H, float eps) {
    __shared__ float lds[8];
    const size_t src = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
    const float* xr = x + src * H;
    const float* dr = delta ? delta + src * H : nullptr;
    auto value = [&](int i) { return dr ? xr[i] + dr[i] : xr[i]; };
    float mean, inv;
    layernorm_row(value, H, eps, lds, mean, inv);
    TOut* o = out + (size_t)blockIdx.x * H;
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = value(i);
        if (resid_out) resid_out[src * H + i] = v;
        o[i] = from_f32<TOut>((v - mean) * inv * w[i] + (b ? b[i] : 0.f));
    }
}

extern "C" int fl_layernorm(const float* x, const float* delta, float* resid_out, const int* rows, const float* w,
                            const float* b, void* out, int out_dtype, int n, int H, float eps, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && x && w && out, "layernorm: bad sizes or a missing tensor");
    FL_CHECK(!(resid_out && rows), "layernorm: the sum is not stored back for picked rows");
    if (n == 0) return 0;
    if (out_dtype == FL_F32) layernorm_kernel<float><<<n, 256, 0, stream>>>(x, delta, resid_out, rows, w, b, (float*)out, H, eps);
    else if (out_dtype == FL_BF16) layernorm_kernel<bf16_t><<<n, 256, 0, stream>>>(x, delta, resid_out, rows, w, b, (bf16_t*)out, H, eps);
    else FL_CHECK(false, "layernorm: unknown dtype %d", out_dtype);
    FL_LAUNCH_CHECK();
    return 0;
}
FL_RECORDABLE(fl_layernorm)

template <typename TC>
__global__ __launch_bounds__(256) void layernorm_add_kernel(const float* __restrict__ delta, const float* __restrict__ w,
                                                            const float* __restrict__ b, float* __restrict__ resid,
                                                            TC* __restrict__ cast, int H, float eps) {
    __shared__ float lds[8];
    const float* dr = delta + (size_t)blockIdx.x * H;
    auto value = [&](int i) { return dr[i]; };
    float mean, inv;
    layernorm_row(value, H, eps, lds, mean, inv);
    float* r = resid + (size_t)blockIdx.x * H;
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = r[i] + ((dr[i] - mean) * inv * w[i] + (b ? b[i] : 0.f));
        r[i] = v;
        if (cast) cast[(size_t)blockIdx.x * H + i] = from_f32<TC>(v);
    }
}

extern "C" int fl_layernorm_add(const float* delta, const float* w, const float* b, float* resid, void* cast, int cast_dtype,
                                int n, int H, float eps, hipStream_t stream) {
    FL_CHECK(n >= 0 && H > 0 && delta && w && resid, "layernorm_add: bad sizes or a missing tensor");
    if (n == 0) return 0;
    if (!cast || cast_dtype == FL_F32) layernorm_add_kernel<float><<<n, 256, 0, stream>>>(delta, w, b, resid, (float*)cast, H, eps);
    else if (cast_dtype == FL_BF16) layernorm_add_kernel<bf16_t><<<n, 256, 0, stream>>>(delta, w, b, resid, (bf16_t*)cast, H, eps);
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
