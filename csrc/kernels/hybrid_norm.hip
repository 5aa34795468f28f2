// Row kernels of the hybrid decoders over an fp32 residual stream:
//   residual_group_norm  x += y (optional); h = grouped RMSNorm(x) * w
//   depth_mix_norm       the end of a depth-averaged layer: store the layer's result,
//                        form the weighted sum of all results so far, norm it for the
//                        next layer -- one pass over the row instead of three kernels
//   head_norm_gate       per-head RMS norm of a recurrence output, weight, sigmoid gate
//   xielu                the xIELU activation
//   gate_proj            a few fp32 gate outputs per row: act(h . w^T + b)
//   residual_norm        x += mult * (add, or RMS-normed add * weight); h = RMSNorm(x) * w
//   gate_mul, relu_sq, side_gate   element-wise epilogues between GEMMs
// All arithmetic is fp32; T is the activation dtype of h / y (bf16, f16 or fp32).
// One workgroup per row; a row is walked twice (sum of squares, then scale), the second
// walk re-reading what the same thread wrote in the first.
#include "common.h"
#include "launch.h"

namespace kgc {

namespace {

constexpr int NT = 256;
constexpr int MAX_GROUPS = 64;

// sum of squares per group -> rsqrt(mean + eps), in rs[0..groups)
template <typename F>
__device__ __forceinline__ void group_scales(F&& value, int W, int groups, float eps, float* rs,
                                             float* scratch) {
  const int gw = W / groups;
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    for (int c = g * gw + threadIdx.x; c < (g + 1) * gw; c += NT) {
      const float v = value(c);
      ss += v * v;
    }
    ss = block_sum<NT>(ss, scratch);
    if (threadIdx.x == 0) rs[g] = 1.f / sqrtf(ss / (float)gw + eps);
  }
  __syncthreads();
}

template <typename T>
__global__ __launch_bounds__(NT) void residual_group_norm_kernel(
    T* __restrict__ out, float* __restrict__ x, const T* __restrict__ y,
    const float* __restrict__ w, int W, int groups, float eps) {
  __shared__ float rs[MAX_GROUPS];
  __shared__ float scratch[NT / 64];
  const int64_t row = blockIdx.x;
  float* xr = x + row * W;
  if (y != nullptr) {
    const T* yr = y + row * W;
    for (int c = threadIdx.x; c < W; c += NT) xr[c] += to_f(yr[c]);
  }
  group_scales([&](int c) { return xr[c]; }, W, groups, eps, rs, scratch);
  const int gw = W / groups;
  T* o = out + row * W;
  for (int c = threadIdx.x; c < W; c += NT) o[c] = from_f<T>(xr[c] * rs[c / gw] * w[c]);
}

// hist [L + 1, Tcap, W]; layer result -> hist[layer + 1]; x = sum_j coef[j] hist[j]
template <typename T>
__global__ __launch_bounds__(NT) void depth_mix_norm_kernel(
    T* __restrict__ out, float* __restrict__ x, float* __restrict__ hist,
    const T* __restrict__ y, const float* __restrict__ coef, const float* __restrict__ w,
    int layer, int64_t hist_stride, int W, int groups, float eps) {
  __shared__ float rs[MAX_GROUPS];
  __shared__ float scratch[NT / 64];
  const int64_t row = blockIdx.x;
  float* xr = x + row * W;
  const T* yr = y + row * W;
  float* hr = hist + row * W;
  const float own = coef[layer + 1];
  for (int c = threadIdx.x; c < W; c += NT) {
    const float r = xr[c] + to_f(yr[c]);
    hr[(int64_t)(layer + 1) * hist_stride + c] = r;
    float acc = 0.f;
    for (int j = 0; j <= layer; ++j) acc += coef[j] * hr[(int64_t)j * hist_stride + c];
    xr[c] = acc + own * r;
  }
  group_scales([&](int c) { return xr[c]; }, W, groups, eps, rs, scratch);
  const int gw = W / groups;
  T* o = out + row * W;
  for (int c = threadIdx.x; c < W; c += NT) o[c] = from_f<T>(xr[c] * rs[c / gw] * w[c]);
}

// grid (rows, H), 64 threads: o fp32 [rows, H * dv]; g [rows, g_stride] (column slice)
template <typename T>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(
    T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ g, int64_t g_stride,
    const float* __restrict__ w, int H, int dv, float eps) {
  const int64_t row = blockIdx.x;
  const int h = blockIdx.y;
  const float* orow = o + (row * H + h) * dv;
  float ss = 0.f;
  for (int c = threadIdx.x; c < dv; c += 64) ss += orow[c] * orow[c];
  ss = wave_sum(ss);
  const float r = 1.f / sqrtf(ss / (float)dv + eps);
  const T* gr = g + row * g_stride + h * dv;
  T* orr = out + (row * H + h) * dv;
  for (int c = threadIdx.x; c < dv; c += 64) {
    const float gate = 1.f / (1.f + expf(-to_f(gr[c])));
    orr[c] = from_f<T>(orow[c] * r * w[h * dv + c] * gate);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void xielu_kernel(T* __restrict__ out, const T* __restrict__ z,
                                                   const float* __restrict__ ab, int64_t n) {
  const float a = ab[0], b = ab[1];
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT) {
    const float v = to_f(z[i]);
    const float r = v > 0.f ? a * v * v + 0.5f * v : b * (expm1f(v) - v) + 0.5f * v;
    out[i] = from_f<T>(r);
  }
}

__device__ __forceinline__ float gate_act(float y, int kind, float cap) {
  if (kind == 0) return 1.f / (1.f + expf(-y));
  if (kind == 3) return y;                            // the plain projection (router logits)
  y = cap * tanhf(y / cap);
  if (kind == 1) return y;
  // logsigmoid(y) = min(y, 0) - log1p(exp(-|y|))
  return fminf(y, 0.f) - log1pf(expf(-fabsf(y)));
}

// Few rows: grid (rows, ceil(N / 4)); the row of h sits in LDS as fp32 and each of the four
// waves computes one output, eight independent 64-column strips at a time so that the
// weight loads of a strip group are all in flight together.
template <typename T>
__global__ __launch_bounds__(NT) void gate_proj_kernel(
    float* __restrict__ out, const T* __restrict__ h, const T* __restrict__ w,
    const float* __restrict__ bias, int W, int N, int kind_a, int kind_b, int split, float cap) {
  extern __shared__ float hrow[];
  const int64_t row = blockIdx.x;
  const T* hr = h + row * W;
  for (int c = threadIdx.x; c < W; c += NT) hrow[c] = to_f(hr[c]);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = blockIdx.y * (NT / 64) + wave;
  if (n >= N) return;
  const T* wr = w + (int64_t)n * W;
  float acc = 0.f;
  for (int c0 = lane; c0 < W; c0 += 64 * 8) {
    float wv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + 64 * u;
      wv[u] = c < W ? to_f(wr[c]) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + 64 * u;
      if (c < W) acc += hrow[c] * wv[u];
    }
  }
  acc = wave_sum(acc);
  if (lane == 0) {
    if (bias != nullptr) acc += bias[n];
    out[row * N + n] = gate_act(acc, n < split ? kind_a : kind_b, cap);
  }
}

// Many rows: a workgroup keeps 8 rows of w in registers (thread t: columns t, t + 256, ...)
// and walks rows bx, bx + gridDim.x, ...; per row each thread multiplies its columns of h
// into 8 partial sums, which meet through wave shuffles and a double-buffered LDS table.
template <typename T, int CPT>
__global__ __launch_bounds__(NT) void gate_proj_rows_kernel(
    float* __restrict__ out, const T* __restrict__ h, const T* __restrict__ w,
    const float* __restrict__ bias, int rows, int W, int N, int kind_a, int kind_b, int split,
    float cap) {
  constexpr int NB = 8;
  __shared__ float red[2][NT / 64][NB];
  const int n0 = blockIdx.y * NB;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float wr[NB][CPT];
#pragma unroll
  for (int n = 0; n < NB; ++n)
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      const int c = threadIdx.x + NT * j;
      wr[n][j] = (n0 + n < N && c < W) ? to_f(w[(int64_t)(n0 + n) * W + c]) : 0.f;
    }
  int it = 0;
  for (int row = blockIdx.x; row < rows; row += gridDim.x, ++it) {
    const T* hr = h + (int64_t)row * W;
    float acc[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) acc[n] = 0.f;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      const int c = threadIdx.x + NT * j;
      const float hv = c < W ? to_f(hr[c]) : 0.f;
#pragma unroll
      for (int n = 0; n < NB; ++n) acc[n] += hv * wr[n][j];
    }
#pragma unroll
    for (int n = 0; n < NB; ++n) {
      const float t = wave_sum(acc[n]);
      if (lane == 0) red[it & 1][wave][n] = t;
    }
    __syncthreads();
    if (threadIdx.x < NB && n0 + threadIdx.x < N) {
      const int n = n0 + threadIdx.x;
      float t = 0.f;
#pragma unroll
      for (int wv = 0; wv < NT / 64; ++wv) t += red[it & 1][wv][threadIdx.x];
      if (bias != nullptr) t += bias[n];
      out[(int64_t)row * N + n] = gate_act(t, n < split ? kind_a : kind_b, cap);
    }
  }
}

}  // namespace

#define KGC_DISPATCH_T(dtype, ...)                          \
  do {                                                      \
    if ((dtype) == DT_BF16) { typedef bf16 T; __VA_ARGS__; } \
    else if ((dtype) == DT_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef float T; __VA_ARGS__; }                  \
  } while (0)

void launch_residual_group_norm(int dtype, void* out, float* x, const void* y, const float* w,
                                int rows, int W, int groups, float eps, hipStream_t s) {
  if (rows <= 0) return;
  KGC_DISPATCH_T(dtype, residual_group_norm_kernel<T><<<rows, NT, 0, s>>>(
      (T*)out, x, (const T*)y, w, W, groups, eps));
}

void launch_depth_mix_norm(int dtype, void* out, float* x, float* hist, const void* y,
                           const float* coef, const float* w, int layer, int64_t hist_stride,
                           int rows, int W, int groups, float eps, hipStream_t s) {
  if (rows <= 0) return;
  KGC_DISPATCH_T(dtype, depth_mix_norm_kernel<T><<<rows, NT, 0, s>>>(
      (T*)out, x, hist, (const T*)y, coef, w, layer, hist_stride, W, groups, eps));
}

void launch_head_norm_gate(int dtype, void* out, const float* o, const void* g, int64_t g_stride,
                           const float* w, int rows, int H, int dv, float eps, hipStream_t s) {
  if (rows <= 0) return;
  KGC_DISPATCH_T(dtype, head_norm_gate_kernel<T><<<dim3(rows, H), 64, 0, s>>>(
      (T*)out, o, (const T*)g, g_stride, w, H, dv, eps));
}

void launch_xielu(int dtype, void* out, const void* z, const float* ab, int64_t n,
                  hipStream_t s) {
  if (n <= 0) return;
  const int grid = (int)std::min<int64_t>((n + NT - 1) / NT, 256 * 32);
  KGC_DISPATCH_T(dtype, xielu_kernel<T><<<grid, NT, 0, s>>>((T*)out, (const T*)z, ab, n));
}

void launch_gate_proj(int dtype, float* out, const void* h, const void* w, const float* bias,
                      int rows, int W, int N, int kind_a, int kind_b, int split, float cap,
                      hipStream_t s) {
  if (rows <= 0) return;
  if (rows >= 1024 && W <= 16 * NT) {
    // enough rows to amortise holding w in registers: 8 outputs per workgroup column
    const dim3 grid(1024, (N + 7) / 8);
#define KGC_GP(C)                                                                      \
  KGC_DISPATCH_T(dtype, gate_proj_rows_kernel<T, C><<<grid, NT, 0, s>>>(               \
      out, (const T*)h, (const T*)w, bias, rows, W, N, kind_a, kind_b, split, cap))
    if (W <= 4 * NT) KGC_GP(4);
    else if (W <= 8 * NT) KGC_GP(8);
    else KGC_GP(16);
#undef KGC_GP
    return;
  }
  const size_t lds = (size_t)W * sizeof(float);
  const dim3 grid(rows, (N + NT / 64 - 1) / (NT / 64));
  KGC_DISPATCH_T(dtype, gate_proj_kernel<T><<<grid, NT, lds, s>>>(
      out, (const T*)h, (const T*)w, bias, W, N, kind_a, kind_b, split, cap));
}

// ---- scaled residual + plain RMS norm, head gate, squared ReLU, side-input gate ----------
namespace {

// x += mult * a, a = add or add / rms(add) * anw; then out = x / rms(x) * w (w null: x;
// out null: none).  out may be x itself (O = float).  A thread owns columns threadIdx.x +
// k NT; with EPT > 0 (W <= EPT * NT) it keeps them in registers, so x and add are read once
// and x written once; EPT = 0 walks the row in passes, re-reading only what it wrote.
template <typename T, typename O, int EPT>
__global__ __launch_bounds__(NT) void residual_norm_kernel(
    O* out, float* x, const T* __restrict__ add, const float* __restrict__ anw,
    const float* __restrict__ w, float mult, int W, float eps) {
  __shared__ float scratch[NT / 64];
  const int64_t row = blockIdx.x;
  float* xr = x + row * W;
  if constexpr (EPT > 0) {
    float xv[EPT];
#pragma unroll
    for (int k = 0; k < EPT; ++k) {
      const int c = threadIdx.x + k * NT;
      xv[k] = c < W ? xr[c] : 0.f;
    }
    if (add != nullptr) {
      const T* ar = add + row * W;
      float av[EPT];
#pragma unroll
      for (int k = 0; k < EPT; ++k) {
        const int c = threadIdx.x + k * NT;
        av[k] = c < W ? to_f(ar[c]) : 0.f;
      }
      if (anw != nullptr) {
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < EPT; ++k) ss += av[k] * av[k];
        ss = block_sum<NT>(ss, scratch);
        const float ra = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
        for (int k = 0; k < EPT; ++k) {
          const int c = threadIdx.x + k * NT;
          if (c < W) av[k] = av[k] * ra * anw[c];
        }
      }
#pragma unroll
      for (int k = 0; k < EPT; ++k) {
        const int c = threadIdx.x + k * NT;
        xv[k] += mult * av[k];
        if (c < W) xr[c] = xv[k];
      }
    }
    if (out == nullptr) return;
    O* o = out + row * W;
    float r = 1.f;
    if (w != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int k = 0; k < EPT; ++k) ss += xv[k] * xv[k];
      ss = block_sum<NT>(ss, scratch);
      r = 1.f / sqrtf(ss / (float)W + eps);
    }
#pragma unroll
    for (int k = 0; k < EPT; ++k) {
      const int c = threadIdx.x + k * NT;
      if (c < W) o[c] = from_f<O>(w != nullptr ? xv[k] * r * w[c] : xv[k]);
    }
    return;
  }
  if (add != nullptr) {
    const T* ar = add + row * W;
    if (anw != nullptr) {
      float ss = 0.f;
      for (int c = threadIdx.x; c < W; c += NT) {
        const float v = to_f(ar[c]);
        ss += v * v;
      }
      ss = block_sum<NT>(ss, scratch);
      const float ra = 1.f / sqrtf(ss / (float)W + eps);
      for (int c = threadIdx.x; c < W; c += NT) xr[c] += mult * (to_f(ar[c]) * ra * anw[c]);
    } else {
      for (int c = threadIdx.x; c < W; c += NT) xr[c] += mult * to_f(ar[c]);
    }
  }
  if (out == nullptr) return;
  O* o = out + row * W;
  if (w == nullptr) {
    for (int c = threadIdx.x; c < W; c += NT) o[c] = from_f<O>(xr[c]);
    return;
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) ss += xr[c] * xr[c];
  ss = block_sum<NT>(ss, scratch);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) o[c] = from_f<O>(xr[c] * r * w[c]);
}

// out [T, H * dv] (row stride so) = o[t, h, :] (strides st, sh) * sigmoid(g[t, h * dv + :])
// (row stride sg) * scale
template <typename T>
__global__ __launch_bounds__(NT) void gate_mul_kernel(
    T* __restrict__ out, int64_t so, const T* __restrict__ o, int64_t st, int64_t sh,
    const T* __restrict__ g, int64_t sg, int H, int dv, float scale) {
  const int64_t t = blockIdx.x;
  const int n = H * dv;
  for (int e = threadIdx.x; e < n; e += NT) {
    const int h = e / dv, c = e - h * dv;
    const float gate = 1.f / (1.f + expf(-to_f(g[t * sg + e])));
    out[t * so + e] = from_f<T>(to_f(o[t * st + h * sh + c]) * gate * scale);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void relu_sq_kernel(T* __restrict__ out, const T* __restrict__ z,
                                                     int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT) {
    const float v = fmaxf(to_f(z[i]), 0.f);
    out[i] = from_f<T>(v * v);
  }
}

// out [T, n] = gelu_tanh(pre [T, n]) * table[ids[t], col0 + :] (table row stride ts)
template <typename T>
__global__ __launch_bounds__(NT) void side_gate_kernel(
    T* __restrict__ out, const T* __restrict__ pre, const int64_t* __restrict__ ids,
    const T* __restrict__ table, int64_t ts, int vocab, int col0, int n) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  if (id < 0 || id >= vocab) id = 0;                  // never read outside the table
  const T* e = table + id * ts + col0;
  for (int c = threadIdx.x; c < n; c += NT) {
    const float z = to_f(pre[t * n + c]);
    const float gl = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    out[t * n + c] = from_f<T>(gl * to_f(e[c]));
  }
}

// The per-token side input of a layer for a few rows (decode steps), one workgroup per row:
//   x += mult * y;  pre = W_g x;  g = gelu_tanh(pre) * table[id, col0 + :];  v = W_p g;
//   x += mult * v / rms(v) * sw;  out = x / rms(x) * w  (w null: no output)
// in one kernel instead of a cast, two small GEMMs, the gate and the add + norm.  Products
// accumulate in fp32 and are rounded to T where the GEMM path rounds (its inputs and
// outputs), so rows that take this kernel agree with rows that take the GEMMs to rounding
// order.  16-bit T, W % 8 == 0, W <= EPT * 1024 threads, n % 8 == 0, n <= 512.
constexpr int SI_NT = 1024, SI_JB = 4;

template <typename T, typename O, int EPT>
__global__ __launch_bounds__(SI_NT) void side_input_rows_kernel(
    O* out, float* x, const T* __restrict__ y, const T* __restrict__ wg,
    const T* __restrict__ wp, const int64_t* __restrict__ ids, const T* __restrict__ table,
    int64_t ts, int vocab, int col0, const float* __restrict__ sw, const float* __restrict__ w,
    float mult, int W, int n, float eps) {
  extern __shared__ float lds[];
  float* xb = lds;                 // [W]: x as the GEMM reads it (rounded to T)
  float* gs = lds + W;             // [n]
  __shared__ float scratch[SI_NT / 64];
  const int64_t row = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* xr = x + row * W;
  float xv[EPT];
#pragma unroll
  for (int k = 0; k < EPT; ++k) {
    const int c = threadIdx.x + k * SI_NT;
    xv[k] = 0.f;
    if (c < W) {
      xv[k] = xr[c] + (y != nullptr ? mult * to_f(y[row * W + c]) : 0.f);
      xb[c] = to_f(from_f<T>(xv[k]));
    }
  }
  __syncthreads();
  int64_t id = ids[row];
  if (id < 0 || id >= vocab) id = 0;
  const T* e = table + id * ts + col0;
  const int chunks = W >> 3;
  // a wave takes SI_JB outputs at a time, their weight rows' loads all in flight
  constexpr int NWV = SI_NT / 64;
  for (int j0 = wave * SI_JB; j0 < n; j0 += NWV * SI_JB) {
    float acc[SI_JB];
#pragma unroll
    for (int b = 0; b < SI_JB; ++b) acc[b] = 0.f;
    for (int ch = lane; ch < chunks; ch += 64) {
      Pack8<T> p[SI_JB];
#pragma unroll
      for (int b = 0; b < SI_JB; ++b)
        p[b].u = *reinterpret_cast<const u32x4*>(wg + (int64_t)min(j0 + b, n - 1) * W + 8 * ch);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float xq = xb[8 * ch + q];
#pragma unroll
        for (int b = 0; b < SI_JB; ++b) acc[b] += xq * to_f(p[b].h[q]);
      }
    }
#pragma unroll
    for (int b = 0; b < SI_JB; ++b) {
      const float tot = wave_sum(acc[b]);
      const int j = j0 + b;
      if (lane == 0 && j < n) {
        const float z = to_f(from_f<T>(tot));
        const float gl = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
        gs[j] = to_f(from_f<T>(gl * to_f(e[j])));
      }
    }
  }
  __syncthreads();
  float vv[EPT], ss = 0.f;
#pragma unroll
  for (int k = 0; k < EPT; ++k) {
    const int c = threadIdx.x + k * SI_NT;
    vv[k] = 0.f;
    if (c < W) {
      const T* pr = wp + (int64_t)c * n;
      float acc = 0.f;
      for (int j0 = 0; j0 < n; j0 += 8) {
        Pack8<T> p;
        p.u = *reinterpret_cast<const u32x4*>(pr + j0);
#pragma unroll
        for (int q = 0; q < 8; ++q) acc += gs[j0 + q] * to_f(p.h[q]);
      }
      vv[k] = to_f(from_f<T>(acc));
      ss += vv[k] * vv[k];
    }
  }
  ss = block_sum<SI_NT>(ss, scratch);
  const float ra = 1.f / sqrtf(ss / (float)W + eps);
  float s2 = 0.f;
#pragma unroll
  for (int k = 0; k < EPT; ++k) {
    const int c = threadIdx.x + k * SI_NT;
    if (c < W) {
      xv[k] += mult * (vv[k] * ra * sw[c]);
      xr[c] = xv[k];
      s2 += xv[k] * xv[k];
    }
  }
  if (out == nullptr || w == nullptr) return;
  s2 = block_sum<SI_NT>(s2, scratch);
  const float r = 1.f / sqrtf(s2 / (float)W + eps);
  O* o = out + row * W;
#pragma unroll
  for (int k = 0; k < EPT; ++k) {
    const int c = threadIdx.x + k * SI_NT;
    if (c < W) o[c] = from_f<O>(xv[k] * r * w[c]);
  }
}

}  // namespace

bool side_input_rows_ok(int dtype, int rows, int W, int n) {
  return (dtype == DT_BF16 || dtype == DT_F16) && rows <= 256 && W % 8 == 0 && W <= 4 * SI_NT &&
         n % 8 == 0 && n <= 512;
}

void launch_side_input_rows(int dtype, int out_dtype, void* out, float* x, const void* y,
                            const void* wg, const void* wp, const int64_t* ids,
                            const void* table, int64_t ts, int vocab, int col0, const float* sw,
                            const float* w, float mult, int rows, int W, int n, float eps,
                            hipStream_t s) {
  if (rows <= 0) return;
  const size_t lds = (size_t)(W + n) * sizeof(float);
#define KGC_SI(T, O, EPT)                                                                     \
  side_input_rows_kernel<T, O, EPT><<<rows, SI_NT, lds, s>>>(                                  \
      (O*)out, x, (const T*)y, (const T*)wg, (const T*)wp, ids, (const T*)table, ts, vocab,   \
      col0, sw, w, mult, W, n, eps)
#define KGC_SI_W(T, O)                     \
  do {                                     \
    if (W <= SI_NT) KGC_SI(T, O, 1);          \
    else if (W <= 2 * SI_NT) KGC_SI(T, O, 2); \
    else KGC_SI(T, O, 4);                     \
  } while (0)
  const bool f32out = out == nullptr || out_dtype == DT_F32;
  if (dtype == DT_BF16) {
    if (f32out) KGC_SI_W(bf16, float); else KGC_SI_W(bf16, bf16);
  } else {
    if (f32out) KGC_SI_W(f16, float); else KGC_SI_W(f16, f16);
  }
#undef KGC_SI_W
#undef KGC_SI
}

void launch_residual_norm(int dtype, int out_dtype, void* out, float* x, const void* add,
                          const float* anw, const float* w, float mult, int rows, int W,
                          float eps, hipStream_t s) {
  if (rows <= 0) return;
#define KGC_RN(O, EPT)                                                          \
  residual_norm_kernel<T, O, EPT><<<rows, NT, 0, s>>>((O*)out, x, (const T*)add, anw, w, mult, \
                                                      W, eps)
#define KGC_RN_W(O)                      \
  do {                                   \
    if (W <= 4 * NT) KGC_RN(O, 4);       \
    else if (W <= 8 * NT) KGC_RN(O, 8);  \
    else if (W <= 16 * NT) KGC_RN(O, 16); \
    else KGC_RN(O, 0);                   \
  } while (0)
  if (out == nullptr || out_dtype == DT_F32) {
    KGC_DISPATCH_T(dtype, KGC_RN_W(float));
  } else {
    KGC_DISPATCH_T(dtype, KGC_RN_W(T));
  }
#undef KGC_RN_W
#undef KGC_RN
}

void launch_gate_mul(int dtype, void* out, int64_t so, const void* o, int64_t st, int64_t sh,
                     const void* g, int64_t sg, int rows, int H, int dv, float scale,
                     hipStream_t s) {
  if (rows <= 0) return;
  KGC_DISPATCH_T(dtype, gate_mul_kernel<T><<<rows, NT, 0, s>>>((T*)out, so, (const T*)o, st, sh,
                                                              (const T*)g, sg, H, dv, scale));
}

void launch_relu_sq(int dtype, void* out, const void* z, int64_t n, hipStream_t s) {
  if (n <= 0) return;
  const int grid = (int)std::min<int64_t>((n + NT - 1) / NT, 256 * 32);
  KGC_DISPATCH_T(dtype, relu_sq_kernel<T><<<grid, NT, 0, s>>>((T*)out, (const T*)z, n));
}

void launch_side_gate(int dtype, void* out, const void* pre, const int64_t* ids,
                      const void* table, int64_t ts, int vocab, int col0, int rows, int n,
                      hipStream_t s) {
  if (rows <= 0) return;
  KGC_DISPATCH_T(dtype, side_gate_kernel<T><<<rows, NT, 0, s>>>(
      (T*)out, (const T*)pre, ids, (const T*)table, ts, vocab, col0, n));
}

}  // namespace kgc
