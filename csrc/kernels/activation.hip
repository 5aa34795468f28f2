// K7 SiLU-and-mul: out[t, i] = silu(x[t, i]) * x[t, I + i] over the fused gate_up
// projection output.  16-byte vector loads/stores (8 halves per lane), one vector
// per thread on a 2-D grid (memory-bound; no index division).
#include "common.h"
#include "launch.h"

namespace kgc {

// grid (ceil(I/8/256), rows): one 16-byte vector per thread, no index division
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(T* __restrict__ out,
                                                       const T* __restrict__ x, int I) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c * 8 >= I) return;
  const int64_t r = blockIdx.y;
  const T* xr = x + r * 2 * I;
  Pack8<T> g, u, o;
  g.u = *reinterpret_cast<const u32x4*>(xr + c * 8);
  u.u = *reinterpret_cast<const u32x4*>(xr + I + c * 8);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float gf = to_f(g.h[j]);
    o.h[j] = from_f<T>(gf / (1.f + __expf(-gf)) * to_f(u.h[j]));
  }
  *reinterpret_cast<u32x4*>(out + r * I + c * 8) = o.u;
}

// any element type and any I (fp32 activations, intermediate sizes that are no multiple of 8)
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_any_kernel(T* __restrict__ out,
                                                           const T* __restrict__ x, int I) {
  const int64_t r = blockIdx.y;
  const T* xr = x + r * 2 * I;
  for (int c = blockIdx.x * 256 + threadIdx.x; c < I; c += gridDim.x * 256) {
    const float gf = to_f(xr[c]);
    out[r * I + c] = from_f<T>(gf / (1.f + expf(-gf)) * to_f(xr[I + c]));
  }
}

void launch_silu_mul(int dtype, void* out, const void* x, int64_t rows, int I, hipStream_t s) {
  if (dtype == DT_F32 || (I & 7)) {
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
      const int64_t n = std::min<int64_t>(rows - r0, 65535);
      const dim3 grid(std::min((I + 255) / 256, 64), (unsigned)n);
      if (dtype == DT_F32)
        silu_mul_any_kernel<float><<<grid, 256, 0, s>>>((float*)out + r0 * I,
                                                        (const float*)x + r0 * 2 * I, I);
      else if (dtype == DT_BF16)
        silu_mul_any_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out + r0 * I,
                                                       (const bf16*)x + r0 * 2 * I, I);
      else
        silu_mul_any_kernel<f16><<<grid, 256, 0, s>>>((f16*)out + r0 * I,
                                                      (const f16*)x + r0 * 2 * I, I);
    }
    return;
  }
  for (int64_t r0 = 0; r0 < rows; r0 += 65535) {   // gridDim.y <= 65535
    const int64_t n = std::min<int64_t>(rows - r0, 65535);
    const dim3 grid(((I >> 3) + 255) / 256, (unsigned)n);
    if (dtype == DT_BF16)
      silu_mul_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out + r0 * I, (const bf16*)x + r0 * 2 * I, I);
    else
      silu_mul_kernel<f16><<<grid, 256, 0, s>>>((f16*)out + r0 * I, (const f16*)x + r0 * 2 * I, I);
  }
}

// ---- PolyNorm, clamped gated activation, scaled embedding + learned positions --------------
namespace {

#define KGC_ACT_DISPATCH_T(dtype, ...)                      \
  do {                                                      \
    if ((dtype) == DT_BF16) { typedef bf16 T; __VA_ARGS__; } \
    else if ((dtype) == DT_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef float T; __VA_ARGS__; }                  \
  } while (0)

// VEC consecutive elements of a row as fp32 (one 16-byte load of 8 halves when VEC = 8)
template <typename T, int VEC>
__device__ __forceinline__ void load_row(const T* p, float (&v)[VEC]) {
  if constexpr (VEC == 8 && !std::is_same_v<T, float>) {
    Pack8<T> t;
    t.u = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_f(t.h[e]);
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = to_f(p[e]);
  }
}

template <typename T, int VEC>
__device__ __forceinline__ void store_row(T* p, const float (&v)[VEC]) {
  if constexpr (VEC == 8 && !std::is_same_v<T, float>) {
    Pack8<T> t;
#pragma unroll
    for (int e = 0; e < 8; ++e) t.h[e] = from_f<T>(v[e]);
    *reinterpret_cast<u32x4*>(p) = t.u;
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) p[e] = from_f<T>(v[e]);
  }
}

// out = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e per row, rms(v) =
// sqrt(mean(v^2) + eps); one workgroup per row, two passes (the second one reads the row
// from cache), fp32 sums.  VEC = 8: 16-bit rows whose length is a multiple of 8.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void polynorm_kernel(T* __restrict__ out,
                                                       const T* __restrict__ z,
                                                       const float* __restrict__ coef, int F,
                                                       float eps) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const T* zr = z + row * F;
  T* orow = out + row * F;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int c = threadIdx.x * VEC; c < F; c += 256 * VEC) {
    float v[VEC];
    load_row<T, VEC>(zr + c, v);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float q = v[e] * v[e];
      s2 += q;
      s4 += q * q;
      s6 += q * q * q;
    }
  }
  s2 = block_sum<256>(s2, scratch);
  s4 = block_sum<256>(s4, scratch);
  s6 = block_sum<256>(s6, scratch);
  const float n = (float)F;
  const float a = coef[0] / sqrtf(s2 / n + eps), b = coef[1] / sqrtf(s4 / n + eps),
              cc = coef[2] / sqrtf(s6 / n + eps), e0 = coef[3];
  for (int c = threadIdx.x * VEC; c < F; c += 256 * VEC) {
    float v[VEC];
    load_row<T, VEC>(zr + c, v);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float x = v[e];
      v[e] = ((cc * x + b) * x + a) * x + e0;
    }
    store_row<T, VEC>(orow + c, v);
  }
}

// x [rows, 2 I] = gate | up  ->  g sigmoid(alpha g) (u + 1), g = min(gate, limit),
// u = clamp(up, -limit, limit)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void swiglu_clamp_kernel(T* __restrict__ out,
                                                           const T* __restrict__ x,
                                                           int64_t rows, int I, float limit,
                                                           float alpha) {
  const int c = (blockIdx.x * 256 + threadIdx.x) * VEC;
  if (c >= I) return;
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
    const T* xr = x + r * 2 * I;
    float g[VEC], u[VEC];
    load_row<T, VEC>(xr + c, g);
    load_row<T, VEC>(xr + I + c, u);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float gv = fminf(g[e], limit), uv = fminf(fmaxf(u[e], -limit), limit);
      g[e] = gv / (1.f + expf(-alpha * gv)) * (uv + 1.f);
    }
    store_row<T, VEC>(out + r * I + c, g);
  }
}

// out fp32 [T, W] = table[ids[t]] * scale + pos[positions[t]]
template <typename T>
__global__ __launch_bounds__(256) void embed_pos_kernel(
    float* __restrict__ out, const int64_t* __restrict__ ids,
    const int64_t* __restrict__ positions, const T* __restrict__ table,
    const float* __restrict__ pos, int W, int vocab, int max_pos, float scale) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t], p = positions[t];
  if (id < 0 || id >= vocab) id = 0;                  // padding rows carry any id
  if (p < 0) p = 0;
  if (p >= max_pos) p = max_pos - 1;
  const T* er = table + id * W;
  const float* pr = pos != nullptr ? pos + p * W : nullptr;
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = to_f(er[c]) * scale;
    if (pr != nullptr) v += pr[c];
    out[t * W + c] = v;
  }
}

}  // namespace

void launch_polynorm(int dtype, void* out, const void* z, const float* coef, int64_t rows, int F,
                     float eps, hipStream_t s) {
  if (rows <= 0 || F <= 0) return;
  const bool vec = dtype != DT_F32 && F % 8 == 0 && reinterpret_cast<uintptr_t>(z) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (vec)
    KGC_ACT_DISPATCH_T(dtype, polynorm_kernel<T, 8><<<rows, 256, 0, s>>>(
        (T*)out, (const T*)z, coef, F, eps));
  else
    KGC_ACT_DISPATCH_T(dtype, polynorm_kernel<T, 1><<<rows, 256, 0, s>>>(
        (T*)out, (const T*)z, coef, F, eps));
}

void launch_swiglu_clamp(int dtype, void* out, const void* x, int64_t rows, int I, float limit,
                         float alpha, hipStream_t s) {
  if (rows <= 0 || I <= 0) return;
  const bool vec = dtype != DT_F32 && I % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int per = 256 * (vec ? 8 : 1);
  const dim3 grid((I + per - 1) / per, (unsigned)(rows < 65535 ? rows : 65535));
  if (vec)
    KGC_ACT_DISPATCH_T(dtype, swiglu_clamp_kernel<T, 8><<<grid, 256, 0, s>>>(
        (T*)out, (const T*)x, rows, I, limit, alpha));
  else
    KGC_ACT_DISPATCH_T(dtype, swiglu_clamp_kernel<T, 1><<<grid, 256, 0, s>>>(
        (T*)out, (const T*)x, rows, I, limit, alpha));
}

void launch_embed_pos(int dtype, float* out, const int64_t* ids, const int64_t* positions,
                      const void* table, const float* pos, int T_, int W, int vocab, int max_pos,
                      float scale, hipStream_t s) {
  if (T_ <= 0) return;
  KGC_ACT_DISPATCH_T(dtype, embed_pos_kernel<T><<<T_, 256, 0, s>>>(
      out, ids, positions, (const T*)table, pos, W, vocab, max_pos, scale));
}

}  // namespace kgc
