// Recurrences whose decay differs per state entry, over per-sequence state slots, all fp32
// past the projections:
//   gla_scan        gated linear attention   S = diag(alpha) S + k v^T,  o = S^T q
//                   with alpha = sigmoid(W_a2 low + b)^(1 / tau) per key channel; the small
//                   second decay projection runs here, so the decay never passes 16 bits
//   selective_scan  S[c, n] = exp(d_c A[c, n]) S[c, n] + d_c x_c B_n,  y_c = S[c, :] . C + D_c x_c
//                   with d = softplus(dt + dt_bias); y * silu(z) * factor in the epilogue
// A step's sequences are its prefill chunks (rows [qsl[i], qsl[i+1]), first position
// seq_lens[i] - rows) followed by its decode rows (one row each, position ctx_lens - 1).  A
// chunk that starts at position 0 starts from zero state; a slot < 0 is a padding row and
// gives zeros.  Prefill chunks and decode rows run the same code, token by token, so a
// position's result does not depend on how the prompt was cut.
//
// Layout: grid (step sequences, heads, column tiles), four waves.  The state of one head is
// S [R, V] (gla: R key channels, V value columns; selective scan: R states, V channels, kept
// in memory as [states, channels] so that a wave's loads are contiguous).  A wave owns 16
// columns (4 when few long sequences have to cover the chip); its lanes are (row group
// rg = lane / columns, column) and a lane keeps rows rg, rg + NRG, ... of its column in
// registers for the whole chunk: S is read and written once per step, and a token's sum over
// rows ends with cross-lane steps inside the wave -- no barrier per token.  Tokens are
// staged in LDS 16 at a time.
#include "common.h"
#include "launch.h"

namespace kgc {

namespace {

constexpr int NT = 256;
constexpr int TB = 16;             // tokens staged per block

struct StepSeq {
  int start, len, pos0, slot;
};

__device__ __forceinline__ StepSeq step_seq(int s, int P, int Tp, const int* qsl,
                                            const int* seq_lens, const int* ctx_lens,
                                            const int* slots) {
  StepSeq q;
  if (s < P) {
    q.start = qsl[s];
    q.len = qsl[s + 1] - q.start;
    q.pos0 = seq_lens[s] - q.len;
  } else {
    q.start = Tp + (s - P);
    q.len = 1;
    q.pos0 = ctx_lens[s - P] - 1;
  }
  q.slot = slots[s];
  return q;
}

__device__ __forceinline__ float softplus_f(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
// ln sigmoid(x) = min(x, 0) - ln(1 + exp(-|x|))
__device__ __forceinline__ float logsigmoid_f(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

// ---- gated linear attention -----------------------------------------------------------------
// proj [T, >= 2 H d + H V] (row stride ps) = q | k | v; low [T, R] (row stride ls) the decay
// bottleneck; a2 fp32 [H d, R], a2b fp32 [H d].
// RPT: rows of S per lane (d <= row groups * RPT); LOGC: log2 of the columns per wave.
template <typename T, int RPT, int LOGC>
__global__ __launch_bounds__(NT) void gla_scan_kernel(
    float* __restrict__ out, const T* __restrict__ proj, int64_t ps, const T* __restrict__ low,
    int64_t ls, const float* __restrict__ a2, const float* __restrict__ a2b,
    float* __restrict__ S, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ ctx_lens, const int* __restrict__ slots, int P, int Tp, int H, int d,
    int V, int R, float inv_tau, int num_slots) {
  constexpr int CW = 1 << LOGC, NRG = 64 >> LOGC;     // columns per wave, row groups per wave
  constexpr int RP = NRG * RPT, CT = CW * (NT / 64);  // rows (padded), columns per workgroup
  constexpr int NG = NT / RP > 0 ? NT / RP : 1;       // token groups of the decay projection
  constexpr int PER = (TB + NG - 1) / NG;             // ... and tokens per thread in it
  extern __shared__ float lds[];
  float* ks = lds;                   // [TB][RP]
  float* qs = ks + TB * RP;          // [TB][RP]
  float* al = qs + TB * RP;          // [TB][RP] decays
  float* vs = al + TB * RP;          // [TB][CT]
  float* lw = vs + TB * CT;          // [TB][R]
  const int s = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, rg = lane >> LOGC;
  const int lc = wave * CW + (lane & (CW - 1)), col = blockIdx.z * CT + lc;
  const bool colok = col < V;
  const StepSeq q = step_seq(s, P, Tp, qsl, seq_lens, ctx_lens, slots);
  const int64_t ow = (int64_t)H * V;
  if (q.slot < 0 || q.slot >= num_slots || q.pos0 < 0 || q.len <= 0) {
    if (rg == 0 && colok)
      for (int t = 0; t < q.len; ++t) out[(int64_t)(q.start + t) * ow + h * V + col] = 0.f;
    return;
  }
  const int qoff = h * d, koff = H * d + h * d, voff = 2 * H * d + h * V;
  float* Sp = S + ((int64_t)q.slot * H + h) * d * V;
  const bool fresh = q.pos0 == 0;
  float Sr[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    Sr[i] = (!fresh && r < d && colok) ? Sp[(int64_t)r * V + col] : 0.f;
  }
  const float qscale = 1.f / sqrtf((float)d);
  for (int t0 = 0; t0 < q.len; t0 += TB) {
    const int nb = min(TB, q.len - t0);
    for (int e = threadIdx.x; e < TB * RP; e += NT) {
      const int tb = e / RP, r = e - tb * RP;
      float kv = 0.f, qv = 0.f;
      if (tb < nb && r < d) {
        const T* row = proj + (int64_t)(q.start + t0 + tb) * ps;
        kv = to_f(row[koff + r]);
        qv = to_f(row[qoff + r]) * qscale;
      }
      ks[e] = kv;
      qs[e] = qv;
    }
    for (int e = threadIdx.x; e < TB * CT; e += NT) {
      const int tb = e / CT, c = blockIdx.z * CT + (e - tb * CT);
      vs[e] = (tb < nb && c < V) ? to_f(proj[(int64_t)(q.start + t0 + tb) * ps + voff + c]) : 0.f;
    }
    for (int e = threadIdx.x; e < TB * R; e += NT) {
      const int tb = e / R, j = e - tb * R;
      lw[e] = tb < nb ? to_f(low[(int64_t)(q.start + t0 + tb) * ls + j]) : 0.f;
    }
    __syncthreads();
    // decays: thread (row r, token group g) keeps its row of a2 in flight once per block
    for (int r = threadIdx.x % RP; r < RP; r += NT) {
      const int g0 = threadIdx.x / RP;
      float acc[PER];
#pragma unroll
      for (int i = 0; i < PER; ++i) acc[i] = 0.f;
      if (r < d) {
        const float* ar = a2 + (int64_t)(h * d + r) * R;
        for (int j = 0; j < R; ++j) {
          const float a = ar[j];
#pragma unroll
          for (int i = 0; i < PER; ++i) {
            const int tb = g0 + i * NG;
            if (tb < TB) acc[i] += a * lw[tb * R + j];
          }
        }
        const float b = a2b[h * d + r];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int tb = g0 + i * NG;
          if (tb < TB) al[tb * RP + r] = expf(logsigmoid_f(acc[i] + b) * inv_tau);
        }
      } else {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int tb = g0 + i * NG;
          if (tb < TB) al[tb * RP + r] = 0.f;
        }
      }
    }
    __syncthreads();
    for (int tb = 0; tb < nb; ++tb) {
      const float vv = vs[tb * CT + lc];
      const float* kp = ks + tb * RP + rg;
      const float* qp = qs + tb * RP + rg;
      const float* ap = al + tb * RP + rg;
      float a0 = 0.f, a1 = 0.f, a2s = 0.f, a3 = 0.f;       // independent chains
#pragma unroll
      for (int i = 0; i < RPT; i += 4) {
        Sr[i] = ap[NRG * i] * Sr[i] + kp[NRG * i] * vv;
        Sr[i + 1] = ap[NRG * (i + 1)] * Sr[i + 1] + kp[NRG * (i + 1)] * vv;
        Sr[i + 2] = ap[NRG * (i + 2)] * Sr[i + 2] + kp[NRG * (i + 2)] * vv;
        Sr[i + 3] = ap[NRG * (i + 3)] * Sr[i + 3] + kp[NRG * (i + 3)] * vv;
        a0 += Sr[i] * qp[NRG * i];
        a1 += Sr[i + 1] * qp[NRG * (i + 1)];
        a2s += Sr[i + 2] * qp[NRG * (i + 2)];
        a3 += Sr[i + 3] * qp[NRG * (i + 3)];
      }
      float y = (a0 + a1) + (a2s + a3);
#pragma unroll
      for (int o = CW; o < 64; o <<= 1) y += __shfl_xor(y, o, 64);
      if (rg == 0 && colok) out[(int64_t)(q.start + t0 + tb) * ow + h * V + col] = y;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    if (r < d && colok) Sp[(int64_t)r * V + col] = Sr[i];
  }
}

// ---- selective scan -------------------------------------------------------------------------
// x, dt [T, I] (contiguous), bc [T, 2 N] (row stride bcs) = B | C, z [T, I] (row stride zs),
// out [T, I] (row stride os), all of type T; At fp32 [N, I] = the transpose of A; state S
// fp32 [slots, N, I].
template <typename T, int RPT, int LOGC>
__global__ __launch_bounds__(NT) void selective_scan_kernel(
    T* __restrict__ out, int64_t os, const T* __restrict__ x, const T* __restrict__ dt,
    const T* __restrict__ bc, int64_t bcs, const float* __restrict__ At,
    const float* __restrict__ dt_bias, const float* __restrict__ dskip,
    const T* __restrict__ z, int64_t zs, float* __restrict__ S, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, const int* __restrict__ ctx_lens,
    const int* __restrict__ slots, int P, int Tp, int I, int N, float out_scale, int num_slots) {
  constexpr int CW = 1 << LOGC, NRG = 64 >> LOGC;
  constexpr int RP = NRG * RPT, CT = CW * (NT / 64);
  extern __shared__ float lds[];
  float* Bs = lds;                   // [TB][RP]
  float* Cs = Bs + TB * RP;          // [TB][RP]
  float* xv = Cs + TB * RP;          // [TB][CT]
  float* dv = xv + TB * CT;          // [TB][CT] step sizes
  const int s = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, rg = lane >> LOGC;
  const int lc = wave * CW + (lane & (CW - 1)), col = blockIdx.z * CT + lc;
  const bool colok = col < I;
  const StepSeq q = step_seq(s, P, Tp, qsl, seq_lens, ctx_lens, slots);
  if (q.slot < 0 || q.slot >= num_slots || q.pos0 < 0 || q.len <= 0) {
    if (rg == 0 && colok)
      for (int t = 0; t < q.len; ++t) out[(int64_t)(q.start + t) * os + col] = from_f<T>(0.f);
    return;
  }
  float* Sp = S + (int64_t)q.slot * N * I;
  const bool fresh = q.pos0 == 0;
  float Sr[RPT], Ar[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    const bool ok = r < N && colok;
    Sr[i] = (!fresh && ok) ? Sp[(int64_t)r * I + col] : 0.f;
    Ar[i] = ok ? At[(int64_t)r * I + col] : 0.f;
  }
  const float Dc = colok ? dskip[col] : 0.f;
  for (int t0 = 0; t0 < q.len; t0 += TB) {
    const int nb = min(TB, q.len - t0);
    for (int e = threadIdx.x; e < TB * RP; e += NT) {
      const int tb = e / RP, r = e - tb * RP;
      float bv = 0.f, cv = 0.f;
      if (tb < nb && r < N) {
        const T* row = bc + (int64_t)(q.start + t0 + tb) * bcs;
        bv = to_f(row[r]);
        cv = to_f(row[N + r]);
      }
      Bs[e] = bv;
      Cs[e] = cv;
    }
    for (int e = threadIdx.x; e < TB * CT; e += NT) {
      const int tb = e / CT, c = blockIdx.z * CT + (e - tb * CT);
      float xx = 0.f, dd = 0.f;
      if (tb < nb && c < I) {
        const int64_t at = (int64_t)(q.start + t0 + tb) * I + c;
        xx = to_f(x[at]);
        dd = softplus_f(to_f(dt[at]) + dt_bias[c]);
      }
      xv[e] = xx;
      dv[e] = dd;
    }
    __syncthreads();
    for (int tb = 0; tb < nb; ++tb) {
      const float xc = xv[tb * CT + lc], d = dv[tb * CT + lc], xd = d * xc;
      const float* bp = Bs + tb * RP + rg;
      const float* cp = Cs + tb * RP + rg;
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; i += 4) {
        Sr[i] = expf(d * Ar[i]) * Sr[i] + bp[NRG * i] * xd;
        Sr[i + 1] = expf(d * Ar[i + 1]) * Sr[i + 1] + bp[NRG * (i + 1)] * xd;
        Sr[i + 2] = expf(d * Ar[i + 2]) * Sr[i + 2] + bp[NRG * (i + 2)] * xd;
        Sr[i + 3] = expf(d * Ar[i + 3]) * Sr[i + 3] + bp[NRG * (i + 3)] * xd;
        a0 += Sr[i] * cp[NRG * i];
        a1 += Sr[i + 1] * cp[NRG * (i + 1)];
        a2 += Sr[i + 2] * cp[NRG * (i + 2)];
        a3 += Sr[i + 3] * cp[NRG * (i + 3)];
      }
      float y = (a0 + a1) + (a2 + a3);
#pragma unroll
      for (int o = CW; o < 64; o <<= 1) y += __shfl_xor(y, o, 64);
      if (rg == 0 && colok) {
        const int64_t t = q.start + t0 + tb;
        const float zv = to_f(z[t * zs + col]);
        out[t * os + col] = from_f<T>((y + Dc * xc) * (zv * sigmoid_f(zv)) * out_scale);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    if (r < N && colok) Sp[(int64_t)r * I + col] = Sr[i];
  }
}

}  // namespace

#define KGC_DS_DISPATCH_T(dtype, ...)                       \
  do {                                                      \
    if ((dtype) == DT_BF16) { typedef bf16 T; __VA_ARGS__; } \
    else if ((dtype) == DT_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef float T; __VA_ARGS__; }                  \
  } while (0)

int decay_scan_max_rows() { return 256; }
int gla_scan_max_rank() { return 128; }      // keeps the staging within 64 KB of LDS

// columns per wave: 16 (a lane holds every 4th row of its column) when that already gives the
// chip two workgroups per CU, else 4 (every 16th row), so that few long sequences still spread
// over the chip
static bool scan_narrow(int seqs, int H, int V) {
  return V <= 4 || (int64_t)seqs * H * ((V + 63) / 64) < 512;
}

static int pow2_at_least(int n, int lo) {
  int p = lo;
  while (p < n) p <<= 1;
  return p;
}

void launch_gla_scan(int dtype, float* out, const void* proj, int64_t ps, const void* low,
                     int64_t ls, const float* a2, const float* a2b, float* S, const int* qsl,
                     const int* seq_lens, const int* ctx_lens, const int* slots, int P, int D,
                     int Tp, int H, int d, int V, int R, float tau, int num_slots,
                     hipStream_t s) {
  if (P + D <= 0) return;
  const bool narrow = scan_narrow(P + D, H, V);
  const int ct = narrow ? 16 : 64, rp = pow2_at_least(d, narrow ? 64 : 16);
  const dim3 grid(P + D, H, (V + ct - 1) / ct);
  const size_t lds = sizeof(float) * (size_t)(3 * TB * rp + TB * ct + TB * R);
#define KGC_GLA_W(RR, L)                                                                     \
  KGC_DS_DISPATCH_T(dtype, gla_scan_kernel<T, RR, L><<<grid, NT, lds, s>>>(                  \
      out, (const T*)proj, ps, (const T*)low, ls, a2, a2b, S, qsl, seq_lens, ctx_lens, slots, P, \
      Tp, H, d, V, R, 1.f / tau, num_slots))
  if (!narrow) {
    if (rp <= 16) KGC_GLA_W(4, 4);
    else if (rp == 32) KGC_GLA_W(8, 4);
    else if (rp == 64) KGC_GLA_W(16, 4);
    else if (rp == 128) KGC_GLA_W(32, 4);
    else KGC_GLA_W(64, 4);
  } else {
    if (rp <= 64) KGC_GLA_W(4, 2);
    else if (rp == 128) KGC_GLA_W(8, 2);
    else KGC_GLA_W(16, 2);
  }
#undef KGC_GLA_W
}

void launch_selective_scan(int dtype, void* out, int64_t os, const void* x, const void* dt,
                           const void* bc, int64_t bcs, const float* At, const float* dt_bias,
                           const float* dskip, const void* z, int64_t zs, float* S,
                           const int* qsl, const int* seq_lens, const int* ctx_lens,
                           const int* slots, int P, int D, int Tp, int I, int N,
                           float out_scale, int num_slots, hipStream_t s) {
  if (P + D <= 0) return;
  const bool narrow = scan_narrow(P + D, 1, I);
  const int ct = narrow ? 16 : 64, rp = pow2_at_least(N, narrow ? 64 : 16);
  const dim3 grid(P + D, 1, (I + ct - 1) / ct);
  const size_t lds = sizeof(float) * (size_t)(2 * TB * rp + 2 * TB * ct);
#define KGC_SEL_W(RR, L)                                                                     \
  KGC_DS_DISPATCH_T(dtype, selective_scan_kernel<T, RR, L><<<grid, NT, lds, s>>>(            \
      (T*)out, os, (const T*)x, (const T*)dt, (const T*)bc, bcs, At, dt_bias, dskip,          \
      (const T*)z, zs, S, qsl, seq_lens, ctx_lens, slots, P, Tp, I, N, out_scale, num_slots))
  if (!narrow) {
    if (rp <= 16) KGC_SEL_W(4, 4);
    else if (rp == 32) KGC_SEL_W(8, 4);
    else if (rp == 64) KGC_SEL_W(16, 4);
    else if (rp == 128) KGC_SEL_W(32, 4);
    else KGC_SEL_W(64, 4);
  } else {
    if (rp <= 64) KGC_SEL_W(4, 2);
    else if (rp == 128) KGC_SEL_W(8, 2);
    else KGC_SEL_W(16, 2);
  }
#undef KGC_SEL_W
}

}  // namespace kgc
