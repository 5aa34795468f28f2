// Windowed attention with kept first tokens over a plain-layout paged cache
// (k [nb, G, bs, dk], v [nb, G, bs, dv]; dk != dv allowed, any sizes), for the hybrid
// decoders.  Rows are addressed through their strides (krs, vrs elements per cache row), so
// the values may be columns of the key rows (one latent cache row per token).  Query i sees key j when j <= i and (i - j < window or j < keep_first);
// window <= 0 means plain causal attention.
//
//   rope_kv_store     rotates q and k on the first `rot` dims of a head (pair i, i + rot/2,
//                     or 2i, 2i + 1; cos / sin from an fp32 table), writes q, and k / v
//                     into the cache
//   window_attention  one wave per (token, query head): the token's visible keys are the
//                     kept first tokens plus the window, walked 64 keys at a time (one key
//                     per lane for the scores, one value column per lane for P.V) with an
//                     online softmax.  Prefill chunks and decode rows of a step take the
//                     same path, so a position's result does not depend on how the prompt
//                     was cut.  Scores, softmax weights and the weighted sum are fp32.
#include "common.h"
#include "launch.h"

namespace kgc {

namespace {

template <typename T>
__global__ __launch_bounds__(256) void rope_kv_store_kernel(
    const T* __restrict__ qkv, int64_t qkv_stride, const int64_t* __restrict__ positions,
    const float* __restrict__ table, int rot, int table_rows, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const int64_t* __restrict__ slots, int H,
    int G, int dk, int dv, int bs, int num_blocks, bool interleaved) {
  const int64_t t = blockIdx.x;
  const T* row = qkv + t * qkv_stride;
  int64_t pos = positions[t];
  if (pos < 0) pos = 0;
  if (pos >= table_rows) pos = table_rows - 1;        // host checks max_pos; never read past
  const float* cs = table != nullptr ? table + pos * rot : nullptr;
  const int half = rot >> 1;
  const int64_t slot = slots[t];
  const bool store = slot >= 0 && slot < (int64_t)num_blocks * bs;
  const int64_t blk = store ? slot / bs : 0, off = store ? slot % bs : 0;
  // q heads then k heads: (H + G) * dk elements, rotated pairwise on the first `rot` dims
  const int nqk = (H + G) * dk;
  for (int e = threadIdx.x; e < nqk; e += 256) {
    const int head = e / dk, i = e - head * dk;
    float v = to_f(row[e]);
    if (i < rot) {
      // pair p: dims (p, p + rot/2), or (2p, 2p + 1) when interleaved
      const int p = interleaved ? i >> 1 : (i < half ? i : i - half);
      const bool first = interleaved ? !(i & 1) : i < half;
      const int ia = interleaved ? 2 * p : p, ib = interleaved ? 2 * p + 1 : half + p;
      const float c = cs[p], sn = cs[half + p];
      const float a = to_f(row[head * dk + ia]), b = to_f(row[head * dk + ib]);
      float oa, ob;
      neox_rot(a, b, c, sn, oa, ob);
      v = first ? oa : ob;
    }
    if (head < H) {
      q_out[(t * H + head) * dk + i] = from_f<T>(v);
    } else if (store) {
      k_cache[((blk * G + (head - H)) * bs + off) * dk + i] = from_f<T>(v);
    }
  }
  if (store) {
    const T* vrow = row + nqk;
    for (int e = threadIdx.x; e < G * dv; e += 256) {
      const int g = e / dv, i = e - g * dv;
      v_cache[((blk * G + g) * bs + off) * dv + i] = vrow[e];
    }
  }
}

// Attention inputs as unit-RMS vectors: qkv fp32 [T, H dk + G dk + G dv] (row stride qs).
// Each head's q and k (qk_unit) and v (v_unit) is divided by sqrt(mean(x^2) + eps); q at
// position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1); q goes to q_out
// [T, H, dk], k and v into the cache.  One wave per head vector, fp32 math.
template <typename T>
__global__ __launch_bounds__(256) void norm_kv_store_kernel(
    const float* __restrict__ qkv, int64_t qs, const int64_t* __restrict__ positions,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int64_t* __restrict__ slots, int H, int G, int dk, int dv, int bs, int num_blocks,
    float eps, bool qk_unit, bool v_unit, float coef, int every) {
  const int64_t t = blockIdx.x;
  const float* row = qkv + t * qs;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int64_t pos = positions[t];
  if (pos < 0) pos = 0;
  const float temp = coef != 0.f ? 1.f + coef * logf((float)((pos + 1) / every) + 1.f) : 1.f;
  const int64_t slot = slots[t];
  const bool store = slot >= 0 && slot < (int64_t)num_blocks * bs;
  const int64_t blk = store ? slot / bs : 0, off = store ? slot % bs : 0;
  for (int hv = wave; hv < H + 2 * G; hv += 4) {
    const bool isq = hv < H, isk = !isq && hv < H + G;
    const int n = hv < H + G ? dk : dv;
    const float* src = row + (hv < H + G ? hv * dk : (H + G) * dk + (hv - H - G) * dv);
    if (!isq && !store) continue;
    float f = isq ? temp : 1.f;
    if (isq || isk ? qk_unit : v_unit) {
      float ss = 0.f;
      for (int i = lane; i < n; i += 64) ss += src[i] * src[i];
      ss = wave_sum(ss);
      f /= sqrtf(ss / (float)n + eps);
    }
    T* dst = isq ? q_out + (t * H + hv) * dk
                 : isk ? k_cache + ((blk * G + (hv - H)) * bs + off) * dk
                       : v_cache + ((blk * G + (hv - H - G)) * bs + off) * dv;
    for (int i = lane; i < n; i += 64) dst[i] = from_f<T>(src[i] * f);
  }
}

constexpr int MAX_DV_PER_LANE = 16;    // dv <= 1024

// scaled score -> cap * tanh(score / cap) when a cap is set
__device__ __forceinline__ float cap_score(float s, float cap) {
  return cap > 0.f ? cap * tanhf(s / cap) : s;
}

// sigmoid of the element-wise output gate at (row t, column c of the concatenated heads)
template <typename T>
__device__ __forceinline__ float elem_gate(const WindowExtra& ex, int64_t t, int c) {
  if (ex.egate == nullptr) return 1.f;
  const float g = to_f(static_cast<const T*>(ex.egate)[t * ex.egs + c]);
  return 1.f / (1.f + expf(-g));
}

// grid (T, H), one wave.  LDS: q row [dk] fp32, p [64], value-row offsets [64].
template <typename T>
__global__ __launch_bounds__(64) void window_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ pbt, const int* __restrict__ ctx_lens, const int* __restrict__ dbt,
    int bt_stride, int P, int Tp, int H, int G, int dk, int dv, int krs, int vrs, int bs,
    int num_blocks, float scale, int window, int keep_first, const float* __restrict__ gate, int kinds,
    WindowExtra ex) {
  extern __shared__ float lds[];
  if (!(kinds & (blockIdx.x < Tp ? 1 : 2))) return;   // rows another kernel of the step owns
  float* qs = lds;                  // [dk]
  float* pw = lds + dk;             // [64]
  int* voff = (int*)(pw + 64);      // [64] (block * G + g) * bs + row
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  T* orow = out + (int64_t)t * ex.ors + h * dv;
  int pos;
  const int* bt;
  if (t < Tp) {
    int lo = 0, hi = P - 1;          // the sequence whose rows [qsl[i], qsl[i+1]) hold t
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
    }
    pos = seq_lens[lo] - (qsl[lo + 1] - qsl[lo]) + (t - qsl[lo]);
    bt = pbt + (int64_t)lo * bt_stride;
  } else {
    const int dd = t - Tp;
    pos = ctx_lens[dd] - 1;
    bt = dbt + (int64_t)dd * bt_stride;
  }
  if (pos < 0 || pos >= bt_stride * bs) {      // a padding row (or nothing to attend)
    for (int c = lane; c < dv; c += 64) orow[c] = from_f<T>(0.f);
    return;
  }
  const T* qrow = q + ((int64_t)t * H + h) * dk;
  for (int c = lane; c < dk; c += 64) qs[c] = to_f(qrow[c]);
  __syncthreads();
  const int lo_w = window > 0 ? max(0, pos - window + 1) : 0;
  const int ns = min(keep_first, lo_w);           // kept first tokens outside the window
  const int total = ns + (pos - lo_w + 1);
  float m = -INFINITY, l = 0.f;
  float acc[MAX_DV_PER_LANE];
#pragma unroll
  for (int u = 0; u < MAX_DV_PER_LANE; ++u) acc[u] = 0.f;
  for (int base = 0; base < total; base += 64) {
    const int idx = base + lane;
    const bool ok = idx < total;
    float s = -INFINITY;
    int ro = 0;
    if (ok) {
      const int j = idx < ns ? idx : lo_w + (idx - ns);
      int b = bt[j / bs];
      if (b < 0 || b >= num_blocks) b = 0;       // never index outside the pool
      ro = (b * G + g) * bs + (j % bs);
      const T* kr = k_cache + (int64_t)ro * krs;
      float d = 0.f;
      for (int c = 0; c < dk; ++c) d += qs[c] * to_f(kr[c]);
      s = cap_score(d * scale, ex.softcap);
    }
    const float mn = fmaxf(m, wave_max(s));
    const float alpha = expf(m - mn);             // m = -inf at first: exp(-inf) = 0
    const float p = ok ? expf(s - mn) : 0.f;
    l = l * alpha + wave_sum(p);
    m = mn;
    __syncthreads();                              // the previous chunk's pw / voff were read
    pw[lane] = p;
    voff[lane] = ro;
    __syncthreads();
    const int cnt = min(64, total - base);
#pragma unroll
    for (int u = 0; u < MAX_DV_PER_LANE; ++u) {
      const int c = lane + 64 * u;
      if (c < dv) {
        float a = acc[u] * alpha;
        for (int jj = 0; jj < cnt; ++jj) a += pw[jj] * to_f(v_cache[(int64_t)voff[jj] * vrs + c]);
        acc[u] = a;
      }
    }
  }
  const float gt = (gate != nullptr ? gate[(int64_t)t * H + h] : 1.f) * ex.out_scale;
  const float inv = gt / l;
#pragma unroll
  for (int u = 0; u < MAX_DV_PER_LANE; ++u) {
    const int c = lane + 64 * u;
    if (c < dv) orow[c] = from_f<T>(acc[u] * inv * elem_gate<T>(ex, t, h * dv + c));
  }
}

// ---- 8 consecutive elements of a cache row as fp32 (16-byte loads; dk % 8 == 0)
template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]) {
  if constexpr (std::is_same_v<T, float>) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    Pack8<T> t;
    t.u = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_f(t.h[e]);
  }
}

// the same 8 elements kept as loaded (4 registers for 16-bit types) until they are used
template <typename T> struct Raw8 { u32x4 u; };
template <> struct Raw8<float> { float4 a, b; };

template <typename T>
__device__ __forceinline__ Raw8<T> load8raw(const T* p) {
  Raw8<T> r;
  if constexpr (std::is_same_v<T, float>) {
    r.a = *reinterpret_cast<const float4*>(p);
    r.b = *reinterpret_cast<const float4*>(p + 4);
  } else {
    r.u = *reinterpret_cast<const u32x4*>(p);
  }
  return r;
}

template <typename T>
__device__ __forceinline__ void cvt8(const Raw8<T>& r, float (&v)[8]) {
  if constexpr (std::is_same_v<T, float>) {
    v[0] = r.a.x; v[1] = r.a.y; v[2] = r.a.z; v[3] = r.a.w;
    v[4] = r.b.x; v[5] = r.b.y; v[6] = r.b.z; v[7] = r.b.w;
  } else {
    Pack8<T> t;
    t.u = r.u;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_f(t.h[e]);
  }
}

template <typename T>
__device__ __forceinline__ void load2(const T* p, float& a, float& b) {
  if constexpr (std::is_same_v<T, float>) {
    const float2 t = *reinterpret_cast<const float2*>(p);
    a = t.x;
    b = t.y;
  } else {
    union { uint32_t u; T h[2]; } t;
    t.u = *reinterpret_cast<const uint32_t*>(p);
    a = to_f(t.h[0]);
    b = to_f(t.h[1]);
  }
}

// Decode rows: one workgroup of 8 waves per (row, kv head, group of up to QH query heads).
// The visible keys (kept first tokens + window) are cut into 64-key chunks dealt round-robin
// to the waves.  In a chunk each lane takes one key: its row is read once (16-byte loads)
// and dotted with every query head of the group (q in LDS as fp32); then each lane takes
// two value columns and walks the chunk's 64 value rows, again once for all heads.  Every
// wave carries its own online-softmax state per head; the eight states merge in LDS in
// wave order (deterministic).  Scores, weights and sums are fp32.
constexpr int DEC_WAVES = 8;          // waves per workgroup (4 when the grid is large)
constexpr int DEC_UMAX = 4;          // value columns per lane: 2 * DEC_UMAX * 64 >= dv

template <typename T, int QH, int NWV>
__global__ __launch_bounds__(64 * NWV) void window_decode_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ ctx_lens, const int* __restrict__ dbt,
    int bt_stride, int Tp, int H, int G, int dk, int dv, int krs, int vrs, int bs, int num_blocks,
    float scale, int window, int keep_first, const float* __restrict__ gate, WindowExtra ex) {
  extern __shared__ float lds[];
  const int dd = blockIdx.x, g = blockIdx.y, qpg = H / G, hq0 = blockIdx.z * QH;
  const int nh = min(QH, qpg - hq0);
  const int t = Tp + dd, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* qs = lds;                                    // [QH][dk]
  float* pb = qs + QH * dk;                           // [waves][QH][64]
  int* ob = (int*)(pb + NWV * QH * 64);         // [waves][64]
  float* mm = (float*)(ob + NWV * 64);          // [waves][QH]
  float* ml = mm + NWV * QH;                    // [waves][QH]
  float* accs = ml + NWV * QH;                  // [QH][dv]
  const int h0 = g * qpg + hq0;                       // first query head of this workgroup
  const int pos = ctx_lens[dd] - 1;
  const int* bt = dbt + (int64_t)dd * bt_stride;
  if (pos < 0 || pos >= bt_stride * bs) {             // a padding row: zeros
    for (int e = threadIdx.x; e < nh * dv; e += 64 * NWV)
      out[(int64_t)t * ex.ors + h0 * dv + e] = from_f<T>(0.f);
    return;
  }
  for (int e = threadIdx.x; e < nh * dk; e += 64 * NWV)
    qs[e] = to_f(q[((int64_t)t * H + h0) * dk + e]);
  for (int e = threadIdx.x; e < QH * dv; e += 64 * NWV) accs[e] = 0.f;
  __syncthreads();
  const int lo_w = window > 0 ? max(0, pos - window + 1) : 0;
  const int ns = min(keep_first, lo_w);
  const int total = ns + (pos - lo_w + 1);
  const int nchunks = (total + 63) >> 6;
  float m[QH], l[QH], acc[QH][DEC_UMAX][2];
#pragma unroll
  for (int h = 0; h < QH; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int u = 0; u < DEC_UMAX; ++u) acc[h][u][0] = acc[h][u][1] = 0.f;
  }
  float* pw = pb + wave * QH * 64;
  int* ow = ob + wave * 64;
  const int lpr = dv >> 3;                 // lanes per value row in the 16-byte path
  const bool vrow = (dv & 7) == 0 && lpr >= 1 && lpr <= 64;
  const bool vpow2 = (lpr & (lpr - 1)) == 0;
  const int kg = vrow ? 64 / lpr : 1;      // lane groups (lanes past kg * lpr idle)
  for (int chunk = wave; chunk < nchunks; chunk += NWV) {
    const int idx = chunk * 64 + lane;
    const bool ok = idx < total;
    float sc[QH];
#pragma unroll
    for (int h = 0; h < QH; ++h) sc[h] = 0.f;
    int ro = 0;
    if (ok) {
      const int j = idx < ns ? idx : lo_w + (idx - ns);
      int b = bt[j / bs];
      if (b < 0 || b >= num_blocks) b = 0;
      ro = (b * G + g) * bs + (j % bs);
      const T* kr = k_cache + (int64_t)ro * krs;
      constexpr int KB = 8;                       // 16-byte pieces of the key row in flight
      for (int c0 = 0; c0 < dk; c0 += 8 * KB) {
        Raw8<T> kraw[KB];
#pragma unroll
        for (int b = 0; b < KB; ++b) {
          const int c = min(c0 + 8 * b, dk - 8);  // clamped: pieces past dk are not used
          kraw[b] = load8raw(kr + c);
        }
#pragma unroll
        for (int b = 0; b < KB; ++b) {
          const int c = c0 + 8 * b;
          if (c < dk) {
            float kv[8];
            cvt8(kraw[b], kv);
#pragma unroll
            for (int h = 0; h < QH; ++h) {
              if (h < nh) {
                const float* qh = qs + h * dk + c;
#pragma unroll
                for (int e = 0; e < 8; ++e) sc[h] += qh[e] * kv[e];
              }
            }
          }
        }
      }
    }
    float alpha[QH];
#pragma unroll
    for (int h = 0; h < QH; ++h) {
      const float sv = ok ? cap_score(sc[h] * scale, ex.softcap) : -INFINITY;
      const float mn = fmaxf(m[h], wave_max(sv));
      alpha[h] = expf(m[h] - mn);
      const float p = ok ? expf(sv - mn) : 0.f;
      l[h] = l[h] * alpha[h] + wave_sum(p);
      m[h] = mn;
      pw[h * 64 + lane] = p;
    }
    ow[lane] = ro;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int cnt = min(64, total - chunk * 64);
    if (vrow) {
      // lpr lanes cover a value row with 16-byte loads; the 64 / lpr lane groups take
      // every (64 / lpr)-th key of the chunk and are summed once, after the last chunk
#pragma unroll
      for (int h = 0; h < QH; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e >> 1][e & 1] *= alpha[h];
      const int cg = lane / lpr, ci = lane - cg * lpr;
      constexpr int VB = std::is_same_v<T, float> ? 4 : 8;    // rows in flight per lane
      for (int j0 = cg < kg ? cg : cnt; j0 < cnt; j0 += VB * kg) {
        Raw8<T> raw[VB];
#pragma unroll
        for (int b = 0; b < VB; ++b) {
          const int jj = min(j0 + b * kg, cnt - 1);            // clamped: weight 0 below
          raw[b] = load8raw(v_cache + (int64_t)ow[jj] * vrs + 8 * ci);
        }
#pragma unroll
        for (int b = 0; b < VB; ++b) {
          const int jj = j0 + b * kg;
          float v8[8];
          cvt8(raw[b], v8);
#pragma unroll
          for (int h = 0; h < QH; ++h) {
            const float p = jj < cnt ? pw[h * 64 + min(jj, 63)] : 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[h][e >> 1][e & 1] += p * v8[e];
          }
        }
      }
    } else {
#pragma unroll
    for (int u = 0; u < DEC_UMAX; ++u) {
      const int c0 = 2 * lane + 128 * u;
      if (c0 < dv) {
        float a0[QH], a1[QH];
#pragma unroll
        for (int h = 0; h < QH; ++h) {
          a0[h] = acc[h][u][0] * alpha[h];
          a1[h] = acc[h][u][1] * alpha[h];
        }
        for (int jj = 0; jj < cnt; ++jj) {
          float v0, v1;
          load2(v_cache + (int64_t)ow[jj] * vrs + c0, v0, v1);
#pragma unroll
          for (int h = 0; h < QH; ++h) {
            const float p = pw[h * 64 + jj];
            a0[h] += p * v0;
            a1[h] += p * v1;
          }
        }
#pragma unroll
        for (int h = 0; h < QH; ++h) {
          acc[h][u][0] = a0[h];
          acc[h][u][1] = a1[h];
        }
      }
    }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) {
#pragma unroll
    for (int h = 0; h < QH; ++h) {
      mm[wave * QH + h] = m[h];
      ml[wave * QH + h] = l[h];
    }
  }
  __syncthreads();
  float f[QH];
#pragma unroll
  for (int h = 0; h < QH; ++h) {
    float M = -INFINITY;
    for (int w = 0; w < NWV; ++w) M = fmaxf(M, mm[w * QH + h]);
    f[h] = m[h] == -INFINITY ? 0.f : expf(m[h] - M);
  }
  if (vrow && vpow2) {
    for (int off = lpr; off < 64; off <<= 1)
#pragma unroll
      for (int h = 0; h < QH; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          acc[h][e >> 1][e & 1] += __shfl_xor(acc[h][e >> 1][e & 1], off, 64);
  } else if (vrow) {
    // lane groups of any width: the first group gathers the others' sums (lanes past it
    // read wrapped lanes; their sums are not used)
#pragma unroll
    for (int h = 0; h < QH; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float own = acc[h][e >> 1][e & 1];
        float tot = own;
        for (int g2 = 1; g2 < kg; ++g2) tot += __shfl(own, (lane + g2 * lpr) & 63, 64);
        acc[h][e >> 1][e & 1] = tot;
      }
  }
  for (int w = 0; w < NWV; ++w) {
    if (vrow) {
      if (wave == w && nchunks > w && lane < lpr) {
#pragma unroll
        for (int h = 0; h < QH; ++h)
#pragma unroll
          for (int e = 0; e < 8; ++e) accs[h * dv + 8 * lane + e] += acc[h][e >> 1][e & 1] * f[h];
      }
    } else if (wave == w && nchunks > w) {
#pragma unroll
      for (int u = 0; u < DEC_UMAX; ++u) {
        const int c0 = 2 * lane + 128 * u;
        if (c0 < dv) {
#pragma unroll
          for (int h = 0; h < QH; ++h) {
            accs[h * dv + c0] += acc[h][u][0] * f[h];
            accs[h * dv + c0 + 1] += acc[h][u][1] * f[h];
          }
        }
      }
    }
    __syncthreads();
  }
  for (int e = threadIdx.x; e < nh * dv; e += 64 * NWV) {
    const int h = e / dv;
    float M = -INFINITY, L = 0.f;
    for (int w = 0; w < NWV; ++w) M = fmaxf(M, mm[w * QH + h]);
    for (int w = 0; w < NWV; ++w) {
      const float mw = mm[w * QH + h];
      if (mw != -INFINITY) L += ml[w * QH + h] * expf(mw - M);
    }
    const float gt = (gate != nullptr ? gate[(int64_t)t * H + h0 + h] : 1.f) * ex.out_scale;
    out[(int64_t)t * ex.ors + h0 * dv + e] =
        from_f<T>(accs[e] * gt / L * elem_gate<T>(ex, t, h0 * dv + e));
  }
}

// Prefill chunks on the matrix cores (16-bit activations).  One workgroup of 4 waves per
// (64 query rows of a chunk, query head); wave w owns rows 16 w .. 16 w + 15.  Keys come in
// 64-key tiles -- first the kept first tokens that lie before the tile's earliest window,
// then the span from that window's start to the last row -- gathered from the pages into
// LDS as K [64][dk + 8] and V^T [dv][64 + 8].  Per tile and wave:
//   S^T = K . Q^T   (v_mfma_f32_16x16x32; the query is lane & 15 in every accumulator, so
//                    the softmax statistics are lane-local up to two shuffles),
//   visibility mask, online softmax in fp32,
//   O^T += V^T . P^T with P^T taken straight from the S^T accumulators (key m of an A row
//                    is 8 (m >> 2) + (m & 3), + 4 for the second tile of a 32-key pair).
// The fp32 weights enter that product as a bf16/f16 pair (value + remainder), two MFMAs,
// so they carry ~16 mantissa bits rather than 8.
constexpr int PFW_BM = 64, PFW_BN = 64, PFW_KPAD = 8, PFW_VPAD = 8;

template <typename T, int KSM, int DTM>
__global__ __launch_bounds__(256, KSM <= 4 ? 3 : 2) void window_prefill_mfma_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ pbt, int bt_stride, const int* __restrict__ work_seq,
    const int* __restrict__ work_blk, int blk_rows, int H, int G, int dk, int dv, int krs,
    int vrs, int bs, int num_blocks, float scale, int window, int keep_first, const float* __restrict__ gate,
    WindowExtra ex) {
  typedef typename Vec8<T>::type V8;
  extern __shared__ float lds_f[];
  T* Ks = reinterpret_cast<T*>(lds_f);                 // [64][dk + 8]
  const int kst = dk + PFW_KPAD, vst = PFW_BN + PFW_VPAD;
  T* Vt = Ks + PFW_BN * kst;                           // [dv][64 + 8]
  const int item = blockIdx.x / (blk_rows / PFW_BM), sub = blockIdx.x % (blk_rows / PFW_BM);
  const int seq = work_seq[item], h = blockIdx.y, g = h / (H / G);
  const int q0 = qsl[seq], qlen = qsl[seq + 1] - q0, ctx0 = seq_lens[seq] - qlen;
  const int r0 = work_blk[item] * blk_rows + sub * PFW_BM;
  if (r0 >= qlen || ctx0 < 0) return;
  const int rows = min(PFW_BM, qlen - r0);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, qd = lane >> 4;
  const int nks = dk >> 5, ndt = dv >> 4;
  const int* bt = pbt + (int64_t)seq * bt_stride;
  const int myrow = r0 + 16 * wave + r16;
  const bool rowok = myrow < qlen;
  const int qpos = ctx0 + myrow;
  // this wave's q fragments: lane (r16, qd) holds dims 32 s + 8 qd .. + 7 of its row
  V8 qf[KSM];
  {
    const T* qrow = q + ((int64_t)(q0 + (rowok ? myrow : r0)) * H + h) * dk;
#pragma unroll
    for (int s2 = 0; s2 < KSM; ++s2) {
      Pack8<T> tq;
      tq.u = u32x4{0u, 0u, 0u, 0u};
      if (s2 < nks && rowok) tq.u = *reinterpret_cast<const u32x4*>(qrow + 32 * s2 + 8 * qd);
      qf[s2] = tq.v;
    }
  }
  f32x4 o[DTM];
#pragma unroll
  for (int t2 = 0; t2 < DTM; ++t2) o[t2] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int p_min = ctx0 + r0, p_max = ctx0 + r0 + rows - 1;
  const int lo_min = window > 0 ? max(0, p_min - window + 1) : 0;
  const int ns = window > 0 ? min(keep_first, lo_min) : 0;
  const int nsink = (ns + PFW_BN - 1) / PFW_BN;
  const int nmain = (p_max - lo_min + PFW_BN) / PFW_BN;
  // the wave's own span of visible keys (tiles outside it are staged but not computed)
  const int wp_lo = ctx0 + r0 + 16 * wave, wp_hi = min(wp_lo + 15, p_max);
  const int w_lo = window > 0 ? max(0, wp_lo - window + 1) : 0;
  const int keyA = 8 * (r16 >> 2) + (r16 & 3);
  const int kchunks = dk >> 3, vchunks = dv >> 3;
  const int bs_shift = (bs & (bs - 1)) == 0 ? __builtin_ctz(bs) : -1;
  auto page_row = [&](int key) -> int64_t {
    const int pg = bs_shift >= 0 ? key >> bs_shift : key / bs;
    const int in = bs_shift >= 0 ? key & (bs - 1) : key - pg * bs;
    int bl = bt[pg];
    if (bl < 0 || bl >= num_blocks) bl = 0;
    return (int64_t)(bl * G + g) * bs + in;
  };
  const int sr = threadIdx.x >> 4, sc = threadIdx.x & 15;     // K staging: 16 lanes per key row
  for (int tile = 0; tile < nsink + nmain; ++tile) {
    const bool sink = tile < nsink;
    const int kb = sink ? tile * PFW_BN : lo_min + (tile - nsink) * PFW_BN;
    const int hi = sink ? min(ns, kb + PFW_BN) : min(p_max + 1, kb + PFW_BN);
    __syncthreads();                         // the previous tile's fragments were read
#pragma unroll
    for (int kq = 0; kq < 4; ++kq) {
      const int ks = sr + 16 * kq, key = kb + ks;
      const T* src = key < hi ? k_cache + page_row(key) * krs : nullptr;
      for (int c = sc; c < kchunks; c += 16) {
        u32x4 val = u32x4{0u, 0u, 0u, 0u};
        if (src != nullptr) val = *reinterpret_cast<const u32x4*>(src + 8 * c);
        *reinterpret_cast<u32x4*>(Ks + ks * kst + 8 * c) = val;
      }
    }
    {
      const int ks = threadIdx.x & (PFW_BN - 1), key = kb + ks;   // a wave's lanes: consecutive keys
      const T* src = key < hi ? v_cache + page_row(key) * vrs : nullptr;
      for (int c = threadIdx.x >> 6; c < vchunks; c += 4) {
        Pack8<T> val;
        val.u = u32x4{0u, 0u, 0u, 0u};
        if (src != nullptr) val.u = *reinterpret_cast<const u32x4*>(src + 8 * c);
#pragma unroll
        for (int e2 = 0; e2 < 8; ++e2) Vt[(8 * c + e2) * vst + ks] = val.h[e2];
      }
    }
    __syncthreads();
    if (16 * wave >= rows) continue;                       // no rows in this wave
    // nothing of this tile is visible to the wave's rows (kept first tokens can sit in a
    // main tile when the earliest window starts before them)
    if (kb > wp_hi || (!sink && hi <= w_lo && kb >= keep_first)) continue;
    // ---- S^T tiles j = 0..3: keys 32 (j >> 1) + keyA + 4 (j & 1)
    f32x4 s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const T* krow = Ks + ((j >> 1) * 32 + keyA + 4 * (j & 1)) * kst + 8 * qd;
      f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s2 = 0; s2 < KSM; ++s2) {
        if (s2 < nks) {
          Pack8<T> fr;
          fr.u = *reinterpret_cast<const u32x4*>(krow + 32 * s2);
          a = mfma16x16x32(fr.v, qf[s2], a);
        }
      }
      s[j] = a;
    }
    // ---- visibility and online softmax (query = lane & 15).  A tile whose 64 keys are
    // all valid, not after the wave's first row and inside the window of its last row is
    // seen in full by every row of the wave: no per-element test.
    const bool full = hi == kb + PFW_BN && kb + PFW_BN - 1 <= wp_lo &&
                      (window <= 0 || wp_hi - kb < window) && wp_lo + 15 == wp_hi;
    float tmax = -INFINITY;
    if (full) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[j][i] = cap_score(s[j][i] * scale, ex.softcap);
          tmax = fmaxf(tmax, s[j][i]);
        }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb + (j >> 1) * 32 + 8 * qd + 4 * (j & 1) + i;
          const bool vis = rowok && key < hi && key <= qpos &&
                           (window <= 0 || qpos - key < window || key < keep_first);
          s[j][i] = vis ? cap_score(s[j][i] * scale, ex.softcap) : -INFINITY;
          tmax = fmaxf(tmax, s[j][i]);
        }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float mn = fmaxf(m, tmax);
    const float alpha = m == -INFINITY ? 0.f : __expf(m - mn);
    m = mn;
    l *= alpha;
    V8 phi[2], plo[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      Pack8<T> ph, pl;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pa = s[2 * kk][i] == -INFINITY ? 0.f : __expf(s[2 * kk][i] - mn);
        const float pb2 = s[2 * kk + 1][i] == -INFINITY ? 0.f : __expf(s[2 * kk + 1][i] - mn);
        l += pa + pb2;
        ph.h[i] = from_f<T>(pa);
        ph.h[4 + i] = from_f<T>(pb2);
        pl.h[i] = from_f<T>(pa - to_f(ph.h[i]));
        pl.h[4 + i] = from_f<T>(pb2 - to_f(ph.h[4 + i]));
      }
      phi[kk] = ph.v;
      plo[kk] = pl.v;
    }
    // ---- O^T += V^T . P^T
#pragma unroll
    for (int t2 = 0; t2 < DTM; ++t2) {
      if (t2 < ndt) {
        f32x4 acc = o[t2] * alpha;
        const T* vrow = Vt + (16 * t2 + r16) * vst + 8 * qd;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          Pack8<T> fr;
          fr.u = *reinterpret_cast<const u32x4*>(vrow + 32 * kk);
          acc = mfma16x16x32(fr.v, phi[kk], acc);
          acc = mfma16x16x32(fr.v, plo[kk], acc);
        }
        o[t2] = acc;
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (rowok) {
    const float gt = (gate != nullptr ? gate[(int64_t)(q0 + myrow) * H + h] : 1.f) * ex.out_scale;
    const float inv = l > 0.f ? gt / l : 0.f;
    T* orow = out + (int64_t)(q0 + myrow) * ex.ors + h * dv;
#pragma unroll
    for (int t2 = 0; t2 < DTM; ++t2) {
      if (t2 < ndt) {
        Pack4<T> w4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          w4.h[i] = from_f<T>(o[t2][i] * inv *
                              elem_gate<T>(ex, q0 + myrow, h * dv + 16 * t2 + 4 * qd + i));
        *reinterpret_cast<u32x2*>(orow + 16 * t2 + 4 * qd) = w4.u;
      }
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

void launch_rope_kv_store(int dtype, const void* qkv, int64_t qkv_stride,
                          const int64_t* positions, const float* table, int rot, int table_rows,
                          void* q_out, void* k_cache, void* v_cache, const int64_t* slots, int T_,
                          int H, int G, int dk, int dv, int bs, int num_blocks, bool interleaved,
                          hipStream_t s) {
  if (T_ <= 0) return;
  KGC_DISPATCH_T(dtype, rope_kv_store_kernel<T><<<T_, 256, 0, s>>>(
      (const T*)qkv, qkv_stride, positions, table, rot, table_rows, (T*)q_out, (T*)k_cache,
      (T*)v_cache, slots, H, G, dk, dv, bs, num_blocks, interleaved));
}

void launch_norm_kv_store(int out_dtype, const float* qkv, int64_t qs, const int64_t* positions,
                          void* q_out, void* k_cache, void* v_cache, const int64_t* slots, int T_,
                          int H, int G, int dk, int dv, int bs, int num_blocks, float eps,
                          bool qk_unit, bool v_unit, float coef, int every, hipStream_t s) {
  if (T_ <= 0) return;
  KGC_DISPATCH_T(out_dtype, norm_kv_store_kernel<T><<<T_, 256, 0, s>>>(
      qkv, qs, positions, (T*)q_out, (T*)k_cache, (T*)v_cache, slots, H, G, dk, dv, bs,
      num_blocks, eps, qk_unit, v_unit, coef, every));
}

int window_attention_max_dv() { return 64 * MAX_DV_PER_LANE; }

void launch_window_attention(int dtype, void* out, const void* q, const void* k_cache,
                             const void* v_cache, const int* qsl, const int* seq_lens,
                             const int* pbt, const int* ctx_lens, const int* dbt, int bt_stride,
                             int P, int Tp, int T_, int H, int G, int dk, int dv, int krs, int vrs,
                             int bs, int num_blocks, float scale, int window, int keep_first,
                             const float* gate, int kinds, WindowExtra ex, hipStream_t s) {
  if (T_ <= 0 || !kinds) return;
  const size_t lds = (size_t)(dk + 128) * sizeof(float);
  KGC_DISPATCH_T(dtype, window_attention_kernel<T><<<dim3(T_, H), 64, lds, s>>>(
      (T*)out, (const T*)q, (const T*)k_cache, (const T*)v_cache, qsl, seq_lens, pbt, ctx_lens,
      dbt, bt_stride, P, Tp, H, G, dk, dv, krs, vrs, bs, num_blocks, scale, window, keep_first,
      gate, kinds, ex));
}

// decode rows on the 8-wave kernel: needs 16-byte key rows (dk % 8 == 0), even dv <= 512
bool window_decode_ok(int dk, int dv, int qpg) {
  (void)qpg;
  return dk % 8 == 0 && dv % 2 == 0 && dv <= 128 * DEC_UMAX;
}

static size_t decode_lds(int QH, int nwv, int dk, int dv) {
  return sizeof(float) * ((size_t)QH * dk + (size_t)nwv * QH * 64 + nwv * 64 + 2 * nwv * QH +
                          (size_t)QH * dv);
}

template <typename T>
static void decode_dispatch(T* out, const T* q, const T* kc, const T* vc, const int* ctx_lens,
                            const int* dbt, int bt_stride, int Tp, int D, int H, int G, int dk,
                            int dv, int krs, int vrs, int bs, int num_blocks, float scale, int window,
                            int keep_first, const float* gate, WindowExtra ex, hipStream_t s) {
  const int qpg = H / G;
  int QH = qpg >= 8 ? 8 : qpg >= 3 ? 4 : qpg;            // heads per workgroup: 1, 2, 4, 8
  // many heads on one key/value group and few rows: smaller head groups, so that the grid
  // still covers the CUs (the groups re-read the rows from L2)
  while (QH > 2 && (int64_t)D * G * ((qpg + QH - 1) / QH) < 256) QH >>= 1;
  const dim3 grid(D, G, (qpg + QH - 1) / QH);
  // 8 waves split a row's keys finest (shortest chain per workgroup); once the grid holds
  // two workgroups per CU, 4-wave workgroups let two of them overlap on a CU instead
  const bool small = (int64_t)grid.x * grid.y * grid.z >= 512;
#define KGC_DEC(N, W)                                                                        \
  window_decode_kernel<T, N, W><<<grid, 64 * W, decode_lds(N, W, dk, dv), s>>>(              \
      out, q, kc, vc, ctx_lens, dbt, bt_stride, Tp, H, G, dk, dv, krs, vrs, bs, num_blocks,     \
      scale, window, keep_first, gate, ex)
#define KGC_DEC2(N) \
  do {              \
    if (small) KGC_DEC(N, 4); else KGC_DEC(N, 8); \
  } while (0)
  if (QH == 8) KGC_DEC2(8);
  else if (QH == 4) KGC_DEC2(4);
  else if (QH == 2) KGC_DEC2(2);
  else KGC_DEC2(1);
#undef KGC_DEC2
#undef KGC_DEC
}

size_t window_decode_lds(int dk, int dv, int qpg) {
  const int QH = qpg >= 8 ? 8 : qpg >= 3 ? 4 : qpg;
  return decode_lds(QH, DEC_WAVES, dk, dv);
}

void launch_window_decode(int dtype, void* out, const void* q, const void* k_cache,
                          const void* v_cache, const int* ctx_lens, const int* dbt,
                          int bt_stride, int Tp, int D, int H, int G, int dk, int dv, int krs,
                          int vrs, int bs, int num_blocks, float scale, int window, int keep_first,
                          const float* gate, WindowExtra ex, hipStream_t s) {
  if (D <= 0) return;
  KGC_DISPATCH_T(dtype, decode_dispatch<T>((T*)out, (const T*)q, (const T*)k_cache,
                                           (const T*)v_cache, ctx_lens, dbt, bt_stride, Tp, D, H,
                                           G, dk, dv, krs, vrs, bs, num_blocks, scale, window, keep_first,
                                           gate, ex, s));
}

size_t window_prefill_mfma_lds(int dk, int dv) {
  return 2 * ((size_t)PFW_BN * (dk + PFW_KPAD) + (size_t)dv * (PFW_BN + PFW_VPAD));
}

// the matrix-core prefill path: 16-bit activations, dk a multiple of 32 (<= 256), dv a
// multiple of 16 (<= 256), both tiles within 64 KB of LDS
bool window_prefill_mfma_ok(int dtype, int dk, int dv) {
  return (dtype == DT_BF16 || dtype == DT_F16) && dk % 32 == 0 && dk <= 256 && dv % 16 == 0 &&
         dv <= 256 && window_prefill_mfma_lds(dk, dv) <= 64 * 1024;
}

template <typename T>
static void prefill_dispatch(T* out, const T* q, const T* kc, const T* vc, const int* qsl,
                             const int* seq_lens, const int* pbt, int bt_stride,
                             const int* work_seq, const int* work_blk, int n_work, int blk_rows,
                             int H, int G, int dk, int dv, int krs, int vrs, int bs, int num_blocks,
                             float scale, int window, int keep_first, const float* gate,
                             WindowExtra ex, hipStream_t s) {
  const dim3 grid(n_work * (blk_rows / PFW_BM), H);
  const size_t lds = window_prefill_mfma_lds(dk, dv);
#define KGC_PF(K, D)                                                                          \
  window_prefill_mfma_kernel<T, K, D><<<grid, 256, lds, s>>>(                                 \
      out, q, kc, vc, qsl, seq_lens, pbt, bt_stride, work_seq, work_blk, blk_rows, H, G, dk,  \
      dv, krs, vrs, bs, num_blocks, scale, window, keep_first, gate, ex)
  if (dk <= 128 && dv <= 128) KGC_PF(4, 8);
  else KGC_PF(8, 16);
#undef KGC_PF
}

void launch_window_prefill_mfma(int dtype, void* out, const void* q, const void* k_cache,
                                const void* v_cache, const int* qsl, const int* seq_lens,
                                const int* pbt, int bt_stride, const int* work_seq,
                                const int* work_blk, int n_work, int blk_rows, int H, int G,
                                int dk, int dv, int krs, int vrs, int bs, int num_blocks, float scale, int window,
                                int keep_first, const float* gate, WindowExtra ex, hipStream_t s) {
  if (n_work <= 0) return;
  if (dtype == DT_BF16)
    prefill_dispatch<bf16>((bf16*)out, (const bf16*)q, (const bf16*)k_cache,
                           (const bf16*)v_cache, qsl, seq_lens, pbt, bt_stride, work_seq,
                           work_blk, n_work, blk_rows, H, G, dk, dv, krs, vrs, bs, num_blocks,
                           scale, window, keep_first, gate, ex, s);
  else
    prefill_dispatch<f16>((f16*)out, (const f16*)q, (const f16*)k_cache, (const f16*)v_cache,
                          qsl, seq_lens, pbt, bt_stride, work_seq, work_blk, n_work, blk_rows, H,
                          G, dk, dv, krs, vrs, bs, num_blocks, scale, window, keep_first, gate, ex, s);
}

// ---- latent attention: cache rows [normed latent | rotary key part] and query rows --------
namespace {

// One workgroup per token.  proj row: per head [d unrotated | r rotary] query columns, then
// the latent pre-activation (rank) and the shared rotary key part (r).  q_lat [H, T, rank]
// holds the unrotated query parts already multiplied into latent space.
//   q_out [T, H, rank + r] = [q_lat | rotated query part]
//   cache row (slot)       = [latent / rms(latent) * nw | rotated key part]
// Rotary pairs are (2i, 2i + 1); table row = cos[r/2] | sin[r/2], fp32.
template <typename T>
__global__ __launch_bounds__(256) void latent_rope_store_kernel(
    T* __restrict__ q_out, const T* __restrict__ proj, int64_t proj_stride,
    const T* __restrict__ q_lat, const int64_t* __restrict__ positions,
    const float* __restrict__ table, int table_rows, const float* __restrict__ nw, float eps,
    T* __restrict__ cache, const int64_t* __restrict__ slots, int64_t cache_rows, int T_, int H,
    int d, int r, int rank) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  const T* row = proj + t * proj_stride;
  int64_t pos = positions[t];
  if (pos < 0) pos = 0;
  if (pos >= table_rows) pos = table_rows - 1;        // host checks max_pos; never read past
  const float* cs = table != nullptr ? table + pos * r : nullptr;
  const int half = r >> 1, dq = d + r, dk = rank + r;
  for (int e = threadIdx.x; e < H * dk; e += 256) {
    const int head = e / dk, i = e - head * dk;
    float v;
    if (i < rank) {
      v = to_f(q_lat[((int64_t)head * T_ + t) * rank + i]);
    } else {
      const int j = i - rank, p = j >> 1;
      const T* qr = row + head * dq + d;
      float oa, ob;
      neox_rot(to_f(qr[2 * p]), to_f(qr[2 * p + 1]), cs[p], cs[half + p], oa, ob);
      v = (j & 1) ? ob : oa;
    }
    q_out[t * H * dk + e] = from_f<T>(v);
  }
  const int64_t slot = slots[t];
  const T* kv = row + (int64_t)H * dq;
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += 256) {
    const float v = to_f(kv[c]);
    ss += v * v;
  }
  ss = block_sum<256>(ss, scratch);
  if (slot < 0 || slot >= cache_rows) return;
  const float rn = 1.f / sqrtf(ss / (float)rank + eps);
  T* crow = cache + slot * dk;
  for (int c = threadIdx.x; c < dk; c += 256) {
    float v;
    if (c < rank) {
      v = to_f(kv[c]) * rn * nw[c];
    } else {
      const int j = c - rank, p = j >> 1;
      float oa, ob;
      neox_rot(to_f(kv[rank + 2 * p]), to_f(kv[rank + 2 * p + 1]), cs[p], cs[half + p], oa, ob);
      v = (j & 1) ? ob : oa;
    }
    crow[c] = from_f<T>(v);
  }
}

}  // namespace

void launch_latent_rope_store(int dtype, void* q_out, const void* proj, int64_t proj_stride,
                              const void* q_lat, const int64_t* positions, const float* table,
                              int table_rows, const float* nw, float eps, void* cache,
                              const int64_t* slots, int64_t cache_rows, int T_, int H, int d,
                              int r, int rank, hipStream_t s) {
  if (T_ <= 0) return;
  KGC_DISPATCH_T(dtype, latent_rope_store_kernel<T><<<T_, 256, 0, s>>>(
      (T*)q_out, (const T*)proj, proj_stride, (const T*)q_lat, positions, table, table_rows, nw,
      eps, (T*)cache, slots, cache_rows, T_, H, d, r, rank));
}

}  // namespace kgc
