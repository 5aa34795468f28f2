// Recurrent halves of parallel mixers (an attention and a recurrence side by side) over
// per-sequence state slots, all fp32 past the projections:
//   causal_conv       per-channel causal convolution over time (+ bias, SiLU); the last
//                     taps - 1 inputs of every sequence are state
//   ssd_scan          the Mamba-2 recurrence  S = a S + d B x^T,  y = S^T C + D x
//   gated_delta_scan  the gated delta rule    S = g S;  u = beta (v - S^T k);  S += k u^T;
//                     o = S^T q   (q, k made unit vectors here)
//   gated_rms_norm    RMS norm in equal parts of a row with a SiLU gate before or after it
// A step's sequences are its prefill chunks (rows [qsl[i], qsl[i+1]), first position
// seq_lens[i] - rows) followed by its decode rows (one row each, position ctx_lens - 1).  A
// chunk that starts at position 0 starts from zero state; a slot < 0 is a padding row and
// gives zeros.  Prefill chunks and decode rows run the same code, token by token, so a
// position's result does not depend on how the prompt was cut.
//
// Scan layout: grid (step sequences, heads, value-column tiles), four waves.  The state of
// one head is S [R, V] (R: state size N or key size d; V: value columns).  A wave owns 16
// columns (4 when few long sequences have to cover the chip: see scan_narrow); its lanes are (row group rg = lane / 16, column lane % 16) and a lane
// keeps rows rg, rg + 4, rg + 8, ... of its column in registers for the whole chunk, so S
// is read and written once per step and a token's sums over rows end with two cross-lane
// steps inside the wave: no barrier per token.  Tokens are staged in LDS 16 at a time.
#include "common.h"
#include "launch.h"

namespace kgc {

namespace {

constexpr int NT = 256;
constexpr int TB = 16;             // tokens staged per block
constexpr int CV_ROWS = 32;        // rows of a chunk per convolution workgroup
constexpr int CV_KMAX = 8;

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

// ---- causal convolution -------------------------------------------------------------------
// grid (n_work * (blk_rows / CV_ROWS) + D, channel tiles): a prefill work item is
// (sequence, block of blk_rows chunk rows), cut into pieces of CV_ROWS rows; one thread walks
// one channel (or four adjacent ones) through its piece with the last K - 1 inputs in
// registers.  Only the piece that
// holds a chunk's first row reads the sequence's state (CV_ROWS >= K - 1), and the same
// thread replaces it afterwards, so no other workgroup touches it meanwhile.
// VEC adjacent channels of one row as fp32 (one 8- or 16-byte load when VEC = 4)
template <typename T, int VEC>
__device__ __forceinline__ void load_channels(const T* p, float (&v)[VEC]) {
  if constexpr (VEC == 1) {
    v[0] = to_f(p[0]);
  } else if constexpr (std::is_same_v<T, float>) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  } else {
    Pack4<T> t;
    t.u = *reinterpret_cast<const u32x2*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = to_f(t.h[e]);
  }
}

template <int VEC>
__device__ __forceinline__ void load_f32(const float* p, float (&v)[VEC]) {
  if constexpr (VEC == 1) {
    v[0] = p[0];
  } else {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  }
}

template <int VEC>
__device__ __forceinline__ void store_f32(float* p, const float (&v)[VEC]) {
  if constexpr (VEC == 1) p[0] = v[0];
  else *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

// VEC adjacent output channels in the output's type (fp32, or the 16-bit input type)
template <typename O, int VEC>
__device__ __forceinline__ void store_out(O* p, const float (&v)[VEC]) {
  if constexpr (std::is_same_v<O, float>) {
    store_f32<VEC>(p, v);
  } else if constexpr (VEC == 1) {
    p[0] = from_f<O>(v[0]);
  } else {
    Pack4<O> t;
#pragma unroll
    for (int e = 0; e < 4; ++e) t.h[e] = from_f<O>(v[e]);
    *reinterpret_cast<u32x2*>(p) = t.u;
  }
}

// VEC: adjacent channels per thread (4 where the column slice, the channel count and the
// row stride allow 8- / 16-byte accesses, else 1)
template <typename T, typename O, int K, int VEC>
__global__ __launch_bounds__(NT) void causal_conv_kernel(
    O* __restrict__ out, const T* __restrict__ x, int64_t xs, const float* __restrict__ w,
    const float* __restrict__ bias, float* __restrict__ state, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, const int* __restrict__ ctx_lens,
    const int* __restrict__ slots, const int* __restrict__ work_seq,
    const int* __restrict__ work_blk, int n_work, int blk_rows, int P, int Tp, int C,
    int num_slots, bool silu) {
  constexpr int KS = K > 1 ? K - 1 : 1;      // state rows (arrays of at least one entry)
  const int subs = blk_rows / CV_ROWS;
  const int item = blockIdx.x;
  int s, r0;
  if (item < n_work * subs) {
    s = work_seq[item / subs];
    r0 = work_blk[item / subs] * blk_rows + (item % subs) * CV_ROWS;
  } else {
    s = P + (item - n_work * subs);
    r0 = 0;
  }
  const StepSeq q = step_seq(s, P, Tp, qsl, seq_lens, ctx_lens, slots);
  const int c = (blockIdx.y * NT + threadIdx.x) * VEC;
  if (c >= C || r0 >= q.len) return;
  const int nrows = min(CV_ROWS, q.len - r0);
  O* orow = out + (int64_t)(q.start + r0) * C + c;
  if (q.slot < 0 || q.slot >= num_slots || q.pos0 < 0) {
    float z[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) z[v] = 0.f;
    for (int r = 0; r < nrows; ++r) store_out<O, VEC>(orow + (int64_t)r * C, z);
    return;
  }
  const bool fresh = q.pos0 == 0;
  float wk[VEC][K], win[KS][VEC], old[KS][VEC], b[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
#pragma unroll
    for (int j = 0; j < K; ++j) wk[v][j] = w[(int64_t)(c + v) * K + j];
    b[v] = bias != nullptr ? bias[c + v] : 0.f;
  }
  float* st = state + (int64_t)q.slot * (K - 1) * C + c;
  const T* xc = x + (int64_t)q.start * xs + c;
  // win[j], j < K - 1: the inputs at chunk row r0 - (K - 1) + j
#pragma unroll
  for (int j = 0; j < K - 1; ++j) {
    const int idx = r0 - (K - 1) + j;
#pragma unroll
    for (int v = 0; v < VEC; ++v) win[j][v] = 0.f;
    if (idx >= 0) load_channels<T, VEC>(xc + (int64_t)idx * xs, win[j]);
    else if (!fresh) load_f32<VEC>(st + (int64_t)(K - 1 + idx) * C, win[j]);
#pragma unroll
    for (int v = 0; v < VEC; ++v) old[j][v] = win[j][v];
  }
  constexpr int RB = VEC == 1 ? 8 : 4;     // rows whose loads are in flight together
  for (int rb = 0; rb < nrows; rb += RB) {
    float in[RB][VEC];
#pragma unroll
    for (int u = 0; u < RB; ++u) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) in[u][v] = 0.f;
      if (rb + u < nrows) load_channels<T, VEC>(xc + (int64_t)(r0 + rb + u) * xs, in[u]);
    }
#pragma unroll
    for (int u = 0; u < RB; ++u) {
      float y[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        float acc = b[v];
#pragma unroll
        for (int j = 0; j < K - 1; ++j) acc += wk[v][j] * win[j][v];
        acc += wk[v][K - 1] * in[u][v];
        y[v] = silu ? acc * sigmoid_f(acc) : acc;
      }
#pragma unroll
      for (int j = 0; j + 1 < K - 1; ++j)
#pragma unroll
        for (int v = 0; v < VEC; ++v) win[j][v] = win[j + 1][v];
      if constexpr (K > 1) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) win[K - 2][v] = in[u][v];
      }
      if (rb + u < nrows) store_out<O, VEC>(orow + (int64_t)(rb + u) * C, y);
    }
  }
  if (r0 == 0) {
    // the chunk's last K - 1 inputs; a chunk shorter than that keeps some of the old ones
#pragma unroll
    for (int i = 0; i < K - 1; ++i) {
      const int idx = q.len - (K - 1) + i;
      float v4[VEC];
      if (idx >= 0) {
        load_channels<T, VEC>(xc + (int64_t)idx * xs, v4);
      } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) v4[v] = 0.f;
#pragma unroll
        for (int j = 0; j < K - 1; ++j)
          if (j == K - 1 + idx) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) v4[v] = old[j][v];
          }
      }
      store_f32<VEC>(st + (int64_t)i * C, v4);
    }
  }
}

// ---- Mamba-2 recurrence ---------------------------------------------------------------------
// xbc fp32 [T, H V + 2 G N] = x | B | C; dt [T, H] (row stride dts) raw step sizes.
// RPT: rows of S per lane (N <= row groups * RPT); LOGC: log2 of the columns per wave.
template <typename T, int RPT, int LOGC>
__global__ __launch_bounds__(NT) void ssd_scan_kernel(
    float* __restrict__ out, const float* __restrict__ xbc, const T* __restrict__ dt,
    int64_t dts, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const float* __restrict__ dskip, float* __restrict__ S, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, const int* __restrict__ ctx_lens,
    const int* __restrict__ slots, int P, int Tp, int H, int V, int N, int G, int num_slots) {
  constexpr int CW = 1 << LOGC, NRG = 64 >> LOGC;     // columns per wave, row groups per wave
  constexpr int RP = NRG * RPT, NTH = NT, CT = CW * (NT / 64);   // rows (padded), threads, columns per workgroup
  extern __shared__ float lds[];
  float* Bs = lds;                   // [TB][RP]
  float* Cs = Bs + TB * RP;          // [TB][RP]
  float* xv = Cs + TB * RP;          // [TB][CT]
  float* sc = xv + TB * CT;          // [TB][2]: decay, step size
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
  const int g = h / (H / G);
  const int64_t cw = (int64_t)H * V + 2 * G * N;
  const int xoff = h * V, boff = H * V + g * N, coff = H * V + G * N + g * N;
  float* Sp = S + ((int64_t)q.slot * H + h) * N * V;
  const bool fresh = q.pos0 == 0;
  float Sr[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    Sr[i] = (!fresh && r < N && colok) ? Sp[(int64_t)r * V + col] : 0.f;
  }
  const float A = expf(a_log[h]), dtb = dt_bias[h], Dh = dskip[h];
  for (int t0 = 0; t0 < q.len; t0 += TB) {
    const int nb = min(TB, q.len - t0);
    for (int e = threadIdx.x; e < TB * RP; e += NTH) {
      const int tb = e / RP, r = e - tb * RP;
      float bv = 0.f, cv = 0.f;
      if (tb < nb && r < N) {
        const float* row = xbc + (int64_t)(q.start + t0 + tb) * cw;
        bv = row[boff + r];
        cv = row[coff + r];
      }
      Bs[e] = bv;
      Cs[e] = cv;
    }
    for (int e = threadIdx.x; e < TB * CT; e += NTH) {
      const int tb = e / CT, c = blockIdx.z * CT + (e - tb * CT);
      xv[e] = (tb < nb && c < V) ? xbc[(int64_t)(q.start + t0 + tb) * cw + xoff + c] : 0.f;
    }
    if (threadIdx.x < TB) {
      const int tb = threadIdx.x;
      float a = 1.f, d = 0.f;
      if (tb < nb) {
        d = softplus_f(to_f(dt[(int64_t)(q.start + t0 + tb) * dts + h]) + dtb);
        a = expf(-A * d);
      }
      sc[2 * tb] = a;
      sc[2 * tb + 1] = d;
    }
    __syncthreads();
    for (int tb = 0; tb < nb; ++tb) {
      const float a = sc[2 * tb], d = sc[2 * tb + 1];
      const float xc = xv[tb * CT + lc], xd = d * xc;
      const float* bp = Bs + tb * RP + rg;
      const float* cp = Cs + tb * RP + rg;
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;       // independent chains
#pragma unroll
      for (int i = 0; i < RPT; i += 4) {
        Sr[i] = a * Sr[i] + bp[NRG * i] * xd;
        Sr[i + 1] = a * Sr[i + 1] + bp[NRG * (i + 1)] * xd;
        Sr[i + 2] = a * Sr[i + 2] + bp[NRG * (i + 2)] * xd;
        Sr[i + 3] = a * Sr[i + 3] + bp[NRG * (i + 3)] * xd;
        a0 += Sr[i] * cp[NRG * i];
        a1 += Sr[i + 1] * cp[NRG * (i + 1)];
        a2 += Sr[i + 2] * cp[NRG * (i + 2)];
        a3 += Sr[i + 3] * cp[NRG * (i + 3)];
      }
      float y = (a0 + a1) + (a2 + a3);
#pragma unroll
      for (int o = CW; o < 64; o <<= 1) y += __shfl_xor(y, o, 64);
      if (rg == 0 && colok)
        out[(int64_t)(q.start + t0 + tb) * ow + h * V + col] = y + Dh * xc;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    if (r < N && colok) Sp[(int64_t)r * V + col] = Sr[i];
  }
}

// ---- gated delta rule -----------------------------------------------------------------------
// qkv fp32 [T, 2 G d + H V] = q | k | v; ba [T, 2 H] (row stride bas): write strength | decay
// pre-activations.  With the token's S_0 = the state before it:
//   S^T k = g S_0^T k,  o = S_new^T q = g S_0^T q + (k . q) u,  S_new = g S_0 + k u^T
// so both sums over rows are taken over S_0 in one pass.
template <typename T, int RPT, int LOGC>
__global__ __launch_bounds__(NT) void gated_delta_scan_kernel(
    float* __restrict__ out, const float* __restrict__ qkv, const T* __restrict__ ba,
    int64_t bas, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    float* __restrict__ S, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ ctx_lens, const int* __restrict__ slots, int P, int Tp, int H,
    int G, int d, int V, int num_slots) {
  constexpr int CW = 1 << LOGC, NRG = 64 >> LOGC;     // columns per wave, row groups per wave
  constexpr int RP = NRG * RPT, NTH = NT, CT = CW * (NT / 64);   // rows (padded), threads, columns per workgroup
  extern __shared__ float lds[];
  float* ks = lds;                   // [TB][RP]
  float* qs = ks + TB * RP;          // [TB][RP]
  float* vs = qs + TB * RP;          // [TB][CT]
  float* sc = vs + TB * CT;          // [TB][3]: decay, write strength, k . q
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
  const int g = h / (H / G);
  const int64_t cw = (int64_t)2 * G * d + (int64_t)H * V;
  const int qoff = g * d, koff = G * d + g * d, voff = 2 * G * d + h * V;
  float* Sp = S + ((int64_t)q.slot * H + h) * d * V;
  const bool fresh = q.pos0 == 0;
  float Sr[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    Sr[i] = (!fresh && r < d && colok) ? Sp[(int64_t)r * V + col] : 0.f;
  }
  const float A = expf(a_log[h]), dtb = dt_bias[h], qscale = 1.f / sqrtf((float)d);
  for (int t0 = 0; t0 < q.len; t0 += TB) {
    const int nb = min(TB, q.len - t0);
    for (int e = threadIdx.x; e < TB * RP; e += NTH) {
      const int tb = e / RP, r = e - tb * RP;
      float kv = 0.f, qv = 0.f;
      if (tb < nb && r < d) {
        const float* row = qkv + (int64_t)(q.start + t0 + tb) * cw;
        kv = row[koff + r];
        qv = row[qoff + r];
      }
      ks[e] = kv;
      qs[e] = qv;
    }
    for (int e = threadIdx.x; e < TB * CT; e += NTH) {
      const int tb = e / CT, c = blockIdx.z * CT + (e - tb * CT);
      vs[e] = (tb < nb && c < V) ? qkv[(int64_t)(q.start + t0 + tb) * cw + voff + c] : 0.f;
    }
    __syncthreads();
    // unit vectors, k . q and the gates: wave w takes tokens w, w + 4, ...
    for (int tb = wave; tb < nb; tb += NT / 64) {
      float sq = 0.f, sk = 0.f, kq = 0.f;
      for (int r = lane; r < RP; r += 64) {
        const float kv = ks[tb * RP + r], qv = qs[tb * RP + r];
        sq += qv * qv;
        sk += kv * kv;
        kq += kv * qv;
      }
      sq = wave_sum(sq);
      sk = wave_sum(sk);
      kq = wave_sum(kq);
      const float qn = qscale / sqrtf(sq + 1e-6f), kn = 1.f / sqrtf(sk + 1e-6f);
      for (int r = lane; r < RP; r += 64) {
        ks[tb * RP + r] *= kn;
        qs[tb * RP + r] *= qn;
      }
      if (lane == 0) {
        const T* row = ba + (int64_t)(q.start + t0 + tb) * bas;
        sc[3 * tb] = expf(-A * softplus_f(to_f(row[H + h]) + dtb));
        sc[3 * tb + 1] = sigmoid_f(to_f(row[h]));
        sc[3 * tb + 2] = kq * qn * kn;
      }
    }
    __syncthreads();
    for (int tb = 0; tb < nb; ++tb) {
      const float gd = sc[3 * tb], beta = sc[3 * tb + 1], kq = sc[3 * tb + 2];
      const float vv = vs[tb * CT + lc];
      const float* kp = ks + tb * RP + rg;
      const float* qp = qs + tb * RP + rg;
      float k0 = 0.f, k1 = 0.f, q0 = 0.f, q1 = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; i += 2) {
        k0 += Sr[i] * kp[NRG * i];
        k1 += Sr[i + 1] * kp[NRG * (i + 1)];
        q0 += Sr[i] * qp[NRG * i];
        q1 += Sr[i + 1] * qp[NRG * (i + 1)];
      }
      float sk = k0 + k1, sq = q0 + q1;
#pragma unroll
      for (int o = CW; o < 64; o <<= 1) {
        sk += __shfl_xor(sk, o, 64);
        sq += __shfl_xor(sq, o, 64);
      }
      const float u = beta * (vv - gd * sk);
#pragma unroll
      for (int i = 0; i < RPT; ++i) Sr[i] = gd * Sr[i] + kp[NRG * i] * u;
      if (rg == 0 && colok)
        out[(int64_t)(q.start + t0 + tb) * ow + h * V + col] = gd * sq + kq * u;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = NRG * i + rg;
    if (r < d && colok) Sp[(int64_t)r * V + col] = Sr[i];
  }
}

// ---- RMS norm with a SiLU gate ----------------------------------------------------------------
// One workgroup per row.  Parts of fewer than 1024 columns: one wave per part (parts dealt
// round-robin); larger parts: the whole workgroup on one part after the other.
template <typename T>
__global__ __launch_bounds__(NT) void gated_rms_norm_kernel(
    T* __restrict__ out, int64_t os, const float* __restrict__ y, const T* __restrict__ gate,
    int64_t gs, const float* __restrict__ w, int n, int groups, float eps, bool gate_first) {
  __shared__ float scratch[NT / 64];
  const int64_t t = blockIdx.x;
  const float* yr = y + t * n;
  const T* gr = gate + t * gs;
  T* orow = out + t * os;
  const int gw = n / groups;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const bool wide = gw >= 1024;
  const int first = wide ? 0 : wave, gstep = wide ? 1 : NT / 64;
  const int c0 = wide ? threadIdx.x : lane, cstep = wide ? NT : 64;
  for (int g = first; g < groups; g += gstep) {
    const int lo = g * gw, hi = lo + gw;
    float ss = 0.f;
    for (int c = lo + c0; c < hi; c += cstep) {
      float v = yr[c];
      if (gate_first) {
        const float gv = to_f(gr[c]);
        v *= gv * sigmoid_f(gv);
      }
      ss += v * v;
    }
    ss = wide ? block_sum<NT>(ss, scratch) : wave_sum(ss);
    const float rn = 1.f / sqrtf(ss / (float)gw + eps);
    for (int c = lo + c0; c < hi; c += cstep) {
      const float gv = to_f(gr[c]);
      const float sg = gv * sigmoid_f(gv);
      const float v = gate_first ? yr[c] * sg * rn * w[c] : yr[c] * rn * w[c] * sg;
      orow[c] = from_f<T>(v);
    }
  }
}

}  // namespace

#define KGC_PM_DISPATCH_T(dtype, ...)                       \
  do {                                                      \
    if ((dtype) == DT_BF16) { typedef bf16 T; __VA_ARGS__; } \
    else if ((dtype) == DT_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef float T; __VA_ARGS__; }                  \
  } while (0)

int causal_conv_max_taps() { return CV_KMAX; }

void launch_causal_conv(int dtype, void* out, bool out_f32, const void* x, int64_t xs,
                        const float* w, const float* bias, float* state, const int* qsl,
                        const int* seq_lens, const int* ctx_lens, const int* slots,
                        const int* work_seq, const int* work_blk, int n_work, int blk_rows, int P,
                        int D, int Tp, int C, int K, int num_slots, bool silu, hipStream_t s) {
  const int items = n_work * (blk_rows / CV_ROWS) + D;
  if (items <= 0 || C <= 0) return;
  // four channels per thread where every access is then an aligned 8- or 16-byte one
  const int el = dtype == DT_F32 ? 4 : 2;
  const bool vec = C % 4 == 0 && xs % 4 == 0 && reinterpret_cast<uintptr_t>(x) % (4 * el) == 0 &&
                   reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(state) % 16 == 0;
  const int per = NT * (vec ? 4 : 1);
  const dim3 grid(items, (C + per - 1) / per);
#define KGC_CV_O(KK, V, O)                                                                   \
  causal_conv_kernel<T, O, KK, V><<<grid, NT, 0, s>>>(                                       \
      (O*)out, (const T*)x, xs, w, bias, state, qsl, seq_lens, ctx_lens, slots, work_seq, work_blk, \
      n_work, blk_rows, P, Tp, C, num_slots, silu)
#define KGC_CV_V(KK, V)                                                                      \
  KGC_PM_DISPATCH_T(dtype, if (out_f32) KGC_CV_O(KK, V, float); else KGC_CV_O(KK, V, T))
#define KGC_CV(KK)                                    \
  do {                                                \
    if (vec) KGC_CV_V(KK, 4); else KGC_CV_V(KK, 1);   \
  } while (0)
  switch (K) {
    case 1: KGC_CV(1); break;
    case 2: KGC_CV(2); break;
    case 3: KGC_CV(3); break;
    case 4: KGC_CV(4); break;
    case 5: KGC_CV(5); break;
    case 6: KGC_CV(6); break;
    case 7: KGC_CV(7); break;
    default: KGC_CV(8); break;
  }
#undef KGC_CV
#undef KGC_CV_V
#undef KGC_CV_O
}

int matrix_scan_max_rows() { return 256; }

static size_t scan_lds(int rows_padded, int cols, int extra) {
  return sizeof(float) * (size_t)(2 * TB * rows_padded + TB * cols + TB * extra);
}

// columns per wave: 16 (a lane holds every 4th row of its column) when that already gives the
// chip two workgroups per CU, else 4 (every 16th row: a quarter of the work per wave and two
// more cross-lane steps per sum), so that few long sequences still spread over the chip
static bool scan_narrow(int seqs, int H, int V) {
  return V <= 4 || (int64_t)seqs * H * ((V + 63) / 64) < 512;
}

static int pow2_at_least(int n, int lo) {
  int p = lo;
  while (p < n) p <<= 1;
  return p;
}

void launch_ssd_scan(int dtype, float* out, const float* xbc, const void* dt, int64_t dts,
                     const float* a_log, const float* dt_bias, const float* dskip, float* S,
                     const int* qsl, const int* seq_lens, const int* ctx_lens, const int* slots,
                     int P, int D, int Tp, int H, int V, int N, int G, int num_slots,
                     hipStream_t s) {
  if (P + D <= 0) return;
  const bool narrow = scan_narrow(P + D, H, V);
  const int ct = narrow ? 16 : 64, rp = pow2_at_least(N, narrow ? 64 : 16);
  const dim3 grid(P + D, H, (V + ct - 1) / ct);
#define KGC_SSD_W(R, L)                                                                      \
  KGC_PM_DISPATCH_T(dtype, ssd_scan_kernel<T, R, L><<<grid, NT, scan_lds(rp, ct, 2), s>>>(   \
      out, xbc, (const T*)dt, dts, a_log, dt_bias, dskip, S, qsl, seq_lens, ctx_lens, slots, P, \
      Tp, H, V, N, G, num_slots))
  // rows per lane = padded rows / row groups (4 wide, 16 narrow); at least 4
  if (!narrow) {
    if (rp <= 16) KGC_SSD_W(4, 4);
    else if (rp == 32) KGC_SSD_W(8, 4);
    else if (rp == 64) KGC_SSD_W(16, 4);
    else if (rp == 128) KGC_SSD_W(32, 4);
    else KGC_SSD_W(64, 4);
  } else {
    if (rp <= 64) KGC_SSD_W(4, 2);
    else if (rp == 128) KGC_SSD_W(8, 2);
    else KGC_SSD_W(16, 2);
  }
#undef KGC_SSD_W
}

void launch_gated_delta_scan(int dtype, float* out, const float* qkv, const void* ba,
                             int64_t bas, const float* a_log, const float* dt_bias, float* S,
                             const int* qsl, const int* seq_lens, const int* ctx_lens,
                             const int* slots, int P, int D, int Tp, int H, int G, int d, int V,
                             int num_slots, hipStream_t s) {
  if (P + D <= 0) return;
  const bool narrow = scan_narrow(P + D, H, V);
  const int ct = narrow ? 16 : 64, rp = pow2_at_least(d, narrow ? 64 : 16);
  const dim3 grid(P + D, H, (V + ct - 1) / ct);
#define KGC_GD_W(R, L)                                                                       \
  KGC_PM_DISPATCH_T(dtype, gated_delta_scan_kernel<T, R, L><<<grid, NT, scan_lds(rp, ct, 3), s>>>( \
      out, qkv, (const T*)ba, bas, a_log, dt_bias, S, qsl, seq_lens, ctx_lens, slots, P, Tp, H, \
      G, d, V, num_slots))
  if (!narrow) {
    if (rp <= 16) KGC_GD_W(4, 4);
    else if (rp == 32) KGC_GD_W(8, 4);
    else if (rp == 64) KGC_GD_W(16, 4);
    else if (rp == 128) KGC_GD_W(32, 4);
    else KGC_GD_W(64, 4);
  } else {
    if (rp <= 64) KGC_GD_W(4, 2);
    else if (rp == 128) KGC_GD_W(8, 2);
    else KGC_GD_W(16, 2);
  }
#undef KGC_GD_W
}

void launch_gated_rms_norm(int dtype, void* out, int64_t os, const float* y, const void* gate,
                           int64_t gs, const float* w, int rows, int n, int groups, float eps,
                           bool gate_first, hipStream_t s) {
  if (rows <= 0) return;
  KGC_PM_DISPATCH_T(dtype, gated_rms_norm_kernel<T><<<rows, NT, 0, s>>>(
      (T*)out, os, y, (const T*)gate, gs, w, n, groups, eps, gate_first));
}

}  // namespace kgc
