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
// rg = lane / columns, column) and a lane keeps the RPT consecutive rows rg RPT .. of its
// column in registers for the whole chunk: S is read and written once per step, a token's
// per-row vectors come from LDS four rows per 16-byte read (a row group's rows lie together,
// groups 16 bytes apart in banks), and a token's sum over rows ends with cross-lane steps
// inside the wave -- no barrier per token.  Tokens are staged in LDS 16 at a time (only the
// tokens present: a decode row stages one).
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

// LDS place of state row r when a lane owns RPT consecutive rows: row groups are padded by
// four floats so that the groups' 16-byte reads fall into different banks
template <int RPT>
__device__ __forceinline__ int lrow(int r) { return r + 4 * (r / RPT); }

__device__ __forceinline__ float4 lds4(const float* p) { return *reinterpret_cast<const float4*>(p); }

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
  constexpr int RPS = RP + 4 * NRG;                   // LDS floats per token and vector
  constexpr int NG = NT / RP > 0 ? NT / RP : 1;       // token groups of the decay projection
  constexpr int PER = (TB + NG - 1) / NG;             // ... and tokens per thread in it
  extern __shared__ float lds[];
  float* ks = lds;                   // [TB][RPS]
  float* qs = ks + TB * RPS;         // [TB][RPS]
  float* al = qs + TB * RPS;         // [TB][RPS] decays
  float* vs = al + TB * RPS;         // [TB][CT]
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
    const int r = rg * RPT + i;
    Sr[i] = (!fresh && r < d && colok) ? Sp[(int64_t)r * V + col] : 0.f;
  }
  const float qscale = 1.f / sqrtf((float)d);
  for (int t0 = 0; t0 < q.len; t0 += TB) {
    const int nb = min(TB, q.len - t0);
    for (int e = threadIdx.x; e < nb * RP; e += NT) {
      const int tb = e / RP, r = e - tb * RP;
      float kv = 0.f, qv = 0.f;
      if (r < d) {
        const T* row = proj + (int64_t)(q.start + t0 + tb) * ps;
        kv = to_f(row[koff + r]);
        qv = to_f(row[qoff + r]) * qscale;
      }
      ks[tb * RPS + lrow<RPT>(r)] = kv;
      qs[tb * RPS + lrow<RPT>(r)] = qv;
    }
    for (int e = threadIdx.x; e < nb * CT; e += NT) {
      const int tb = e / CT, c = blockIdx.z * CT + (e - tb * CT);
      vs[e] = c < V ? to_f(proj[(int64_t)(q.start + t0 + tb) * ps + voff + c]) : 0.f;
    }
    for (int e = threadIdx.x; e < nb * R; e += NT) {
      const int tb = e / R, j = e - tb * R;
      lw[e] = to_f(low[(int64_t)(q.start + t0 + tb) * ls + j]);
    }
    __syncthreads();
    // decays: thread (row r, token group g0) reads its row of a2 once per block of tokens
    {
      const int r = threadIdx.x % RP, g0 = threadIdx.x / RP;
      if (g0 < NG && g0 < nb) {
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
              if (tb < nb) acc[i] += a * lw[tb * R + j];
            }
          }
        }
        const float b = r < d ? a2b[h * d + r] : 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int tb = g0 + i * NG;
          if (tb < nb)
            al[tb * RPS + lrow<RPT>(r)] = r < d ? expf(logsigmoid_f(acc[i] + b) * inv_tau) : 0.f;
        }
      }
    }
    __syncthreads();
    for (int tb = 0; tb < nb; ++tb) {
      const float vv = vs[tb * CT + lc];
      const int base = tb * RPS + rg * (RPT + 4);
      float a0 = 0.f, a1 = 0.f, a2s = 0.f, a3 = 0.f;       // independent chains
#pragma unroll
      for (int i = 0; i < RPT; i += 4) {
        const float4 av = lds4(al + base + i), kv = lds4(ks + base + i), qv = lds4(qs + base + i);
        Sr[i] = av.x * Sr[i] + kv.x * vv;
        Sr[i + 1] = av.y * Sr[i + 1] + kv.y * vv;
        Sr[i + 2] = av.z * Sr[i + 2] + kv.z * vv;
        Sr[i + 3] = av.w * Sr[i + 3] + kv.w * vv;
        a0 += Sr[i] * qv.x;
        a1 += Sr[i + 1] * qv.y;
        a2s += Sr[i + 2] * qv.z;
        a3 += Sr[i + 3] * qv.w;
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
    const int r = rg * RPT + i;
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
  constexpr int RPS = RP + 4 * NRG;
  extern __shared__ float lds[];
  float* Bs = lds;                   // [TB][RPS]
  float* Cs = Bs + TB * RPS;         // [TB][RPS]
  float* xv = Cs + TB * RPS;         // [TB][CT]
  float* dv = xv + TB * CT;          // [TB][CT] step sizes
  float* gz = dv + TB * CT;          // [TB][CT] silu(z) * out_scale
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
  // Ar: A times log2(e), so that exp(d A) is one v_exp_f32 of d * Ar (d A <= 0: no overflow,
  // and a result below the normal range is a decay of zero either way)
  float Sr[RPT], Ar[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg * RPT + i;
    const bool ok = r < N && colok;
    Sr[i] = (!fresh && ok) ? Sp[(int64_t)r * I + col] : 0.f;
    Ar[i] = ok ? At[(int64_t)r * I + col] * 1.4426950408889634f : 0.f;
  }
  const float Dc = colok ? dskip[col] : 0.f;
  for (int t0 = 0; t0 < q.len; t0 += TB) {
    const int nb = min(TB, q.len - t0);
    for (int e = threadIdx.x; e < nb * RP; e += NT) {
      const int tb = e / RP, r = e - tb * RP;
      float bv = 0.f, cv = 0.f;
      if (r < N) {
        const T* row = bc + (int64_t)(q.start + t0 + tb) * bcs;
        bv = to_f(row[r]);
        cv = to_f(row[N + r]);
      }
      Bs[tb * RPS + lrow<RPT>(r)] = bv;
      Cs[tb * RPS + lrow<RPT>(r)] = cv;
    }
    for (int e = threadIdx.x; e < nb * CT; e += NT) {
      const int tb = e / CT, c = blockIdx.z * CT + (e - tb * CT);
      float xx = 0.f, dd = 0.f, gg = 0.f;
      if (c < I) {
        const int64_t t = q.start + t0 + tb;
        xx = to_f(x[t * I + c]);
        dd = softplus_f(to_f(dt[t * I + c]) + dt_bias[c]);
        const float zv = to_f(z[t * zs + c]);
        gg = zv * sigmoid_f(zv) * out_scale;
      }
      xv[e] = xx;
      dv[e] = dd;
      gz[e] = gg;
    }
    __syncthreads();
    for (int tb = 0; tb < nb; ++tb) {
      const float xc = xv[tb * CT + lc], d = dv[tb * CT + lc], xd = d * xc;
      const int base = tb * RPS + rg * (RPT + 4);
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; i += 4) {
        const float4 bv = lds4(Bs + base + i), cv = lds4(Cs + base + i);
        Sr[i] = __builtin_amdgcn_exp2f(d * Ar[i]) * Sr[i] + bv.x * xd;
        Sr[i + 1] = __builtin_amdgcn_exp2f(d * Ar[i + 1]) * Sr[i + 1] + bv.y * xd;
        Sr[i + 2] = __builtin_amdgcn_exp2f(d * Ar[i + 2]) * Sr[i + 2] + bv.z * xd;
        Sr[i + 3] = __builtin_amdgcn_exp2f(d * Ar[i + 3]) * Sr[i + 3] + bv.w * xd;
        a0 += Sr[i] * cv.x;
        a1 += Sr[i + 1] * cv.y;
        a2 += Sr[i + 2] * cv.z;
        a3 += Sr[i + 3] * cv.w;
      }
      float y = (a0 + a1) + (a2 + a3);
#pragma unroll
      for (int o = CW; o < 64; o <<= 1) y += __shfl_xor(y, o, 64);
      if (rg == 0 && colok)
        out[(int64_t)(q.start + t0 + tb) * os + col] = from_f<T>((y + Dc * xc) * gz[tb * CT + lc]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg * RPT + i;
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
  bool narrow = scan_narrow(P + D, H, V);
  // the narrow form pads 16 row groups; it has to fit 64 KB of LDS with the decay bottleneck
  if (narrow && sizeof(float) * (size_t)(3 * TB * (pow2_at_least(d, 64) + 64) + TB * 16 + TB * R) >
                    (size_t)64 * 1024)
    narrow = false;
  const int ct = narrow ? 16 : 64, rp = pow2_at_least(d, narrow ? 64 : 16);
  const int rps = rp + 4 * (narrow ? 16 : 4);
  const dim3 grid(P + D, H, (V + ct - 1) / ct);
  const size_t lds = sizeof(float) * (size_t)(3 * TB * rps + TB * ct + TB * R);
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
  const int rps = rp + 4 * (narrow ? 16 : 4);
  const dim3 grid(P + D, 1, (I + ct - 1) / ct);
  const size_t lds = sizeof(float) * (size_t)(2 * TB * rps + 3 * TB * ct);
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
