// Softmax attention on the paged cache with the pieces several decoder designs combine freely:
//   * per-head RMS norms of queries and keys with a learned weight, then a rotation of the first `rot` values of a
//     head, value i paired with value i + rot / 2 (half-split) or value 2i with 2i + 1 (neighbours), angles from an
//     fp32 cos | sin table;
//   * a query temperature: queries at position p times 1 + coef * ln(floor((p + 1) / every) + 1);
//   * value mixing: v <- (1 - lam) v + lam v_first with the values another layer made of the same token, before the
//     cache write;
//   * scores squashed by cap * tanh(score / cap); a learned bias per (query - key distance, head) from a table whose
//     last row serves every larger distance;
//   * key and value widths of their own (D, Dv), grouped query heads;
//   * `maps` score maps per head over the same values (maps = 2: differential attention, o = a1 - lam * a2, divided
//     by its root mean square over Dv and scaled);
//   * masks: causal, and on top a sliding window (i - j < window) and / or chunks counted from the sequence's start
//     (j / chunk == i / chunk);
//   * a sink per head: exp(sink[h]) joins the softmax denominator, with no key and no value;
//   * an output gate: the result times the sigmoid of a second projection.
//
// Cache layout: k_cache [blocks, G, bs, maps * D] (a head's maps side by side in one row), v_cache [blocks, G, Dv, bs].
// For the matrix-core kernels of attention.hip every map is a key head of its own instead (`by_map`): k_cache
// [blocks, G * maps, bs, D], queries ordered (key head, map, head inside the group), so that query row q reads key
// head q / (H / G) and that key head k reads value head k / maps; vda_map_combine folds their output.
//
//   vda_qk_norm_rope_cache         per token: norms, rotation, the query rows out, key rows and values into the cache
//   vda_map_combine                the epilogue of the matrix-core path: maps' combination, its norm, the gate
//   vda_masked_softmax_attention   plain fp32 arithmetic for any sizes and types: one workgroup per (sequence, tile of
//                                  query tokens, group of heads that share a key / value head) walks the visible keys
//                                  in tiles through LDS with a running maximum and sum per row; keys outside the mask
//                                  of the tile's first query are never loaded.  Prompts, portions and single decoded
//                                  tokens are one code path; keys are added in a fixed order per (token, head, map),
//                                  so a result does not depend on how a prompt was cut or batched.
#include "common.h"

// options of the per-token kernel beyond norms and rotation (zero / null: off)
struct QkExtras {
  int neighbours;          // rotation pairs value 2i with 2i + 1 instead of i with i + rot / 2
  float q_coef;            // query temperature: 1 + q_coef * ln(floor((p + 1) / q_every) + 1)
  int q_every;             //   (q_every <= 0: none)
  const void* v_first;     // [T, G * Dv] values of the same tokens from an earlier layer, or null
  long v_first_stride;
  const float* v_lam;      // one value: v <- (1 - lam) v + lam v_first
};

__device__ __forceinline__ float query_temperature(const QkExtras& x, long p) {
  if (x.q_every <= 0) return 1.f;
  return 1.f + x.q_coef * logf((float)((p + 1) / x.q_every + 1));
}

template <typename T>
__device__ __forceinline__ T mixed_value(const QkExtras& x, T v, long t, int e) {
  if (!x.v_first) return v;
  const float lam = *x.v_lam;
  return (T)((1.f - lam) * (float)v + lam * (float)((const T*)x.v_first)[t * x.v_first_stride + e]);
}

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_cache_kernel(
    T* __restrict__ qn, const T* __restrict__ qkv, long qkv_stride, const float* __restrict__ q_w,
    const float* __restrict__ k_w, const float* __restrict__ cos_sin, const long* __restrict__ positions,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const long* __restrict__ slot_mapping, int H, int G, int D,
    int Dv, int maps, int rot, int bs, float eps, int by_map, const QkExtras x) {
  const long t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* row = qkv + t * qkv_stride;
  const int half = rot / 2;
  const float* cs = rot > 0 ? cos_sin + positions[t] * (long)rot : nullptr;
  const long slot = slot_mapping[t];
  const float qt = query_temperature(x, positions[t]);
  const int nq = H * maps, nk = G * maps;
  // one wave per D-wide unit: the query maps first, then the key maps
  for (int u = wave; u < nq + nk; u += 4) {
    const bool is_q = u < nq;
    const T* src = row + (long)u * D;             // q units and k units are contiguous in the row
    const float* w = is_q ? q_w : k_w;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float v = (float)src[d];
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float rs = 1.f / sqrtf(ss / (float)D + eps);
    T* dst;
    if (is_q) {
      int uo = u;                                 // query unit = head * maps + map
      if (by_map) {                               // ... or (key head, map, head inside its group)
        const int R = H / G, h = u / maps, mp = u % maps;
        uo = ((h / R) * maps + mp) * R + h % R;
      }
      dst = qn + (t * nq + uo) * (long)D;
    } else {
      if (slot < 0) continue;
      const int uk = u - nq;                      // key unit = head * maps + map
      const int g = uk / maps, mp = uk % maps;
      dst = by_map ? k_cache + (((slot / bs) * nk + uk) * (long)bs + slot % bs) * (long)D
                   : k_cache + (((slot / bs) * G + g) * (long)bs + slot % bs) * (long)(maps * D) + (long)mp * D;
    }
    for (int d = lane; d < D; d += 64) {
      float v = (float)src[d] * rs * w[d];
      if (d < rot) {
        const bool first = x.neighbours ? !(d & 1) : d < half;
        const int i = x.neighbours ? d >> 1 : (d < half ? d : d - half);
        const int pd = x.neighbours ? d ^ 1 : (d < half ? d + half : d - half);
        const float o = (float)src[pd] * rs * w[pd];
        const float co = cs[i], si = cs[half + i];
        v = first ? v * co - o * si : v * co + o * si;
      }
      dst[d] = (T)(is_q ? v * qt : v);
    }
  }
  if (slot >= 0) {
    const T* vsrc = row + (long)(nq + nk) * D;
    T* vdst = v_cache + (slot / bs) * (long)G * Dv * bs + slot % bs;      // [blocks, G, Dv, bs]
    for (int e = tid; e < G * Dv; e += 256) vdst[(long)e * bs] = mixed_value<T>(x, vsrc[e], t, e);
  }
}

// The same with 8 consecutive values per lane (16-byte accesses for 16-bit rows): LPU = D / 8 lanes share a unit, so a
// workgroup takes 256 / LPU units at a time; the pair partner of a lane's values sits in the lane rot / 16 further on
// (or back) and arrives by a shuffle.  For D in {32, 64, 128, 256}, rot / 2 a multiple of 8, rows 16-byte aligned.
template <typename T, int LPU>
__global__ __launch_bounds__(256) void qk_norm_rope_cache_vec_kernel(
    T* __restrict__ qn, const T* __restrict__ qkv, long qkv_stride, const float* __restrict__ q_w,
    const float* __restrict__ k_w, const float* __restrict__ cos_sin, const long* __restrict__ positions,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const long* __restrict__ slot_mapping, int H, int G, int Dv,
    int maps, int rot, int bs, float eps, int by_map, const QkExtras xo) {
  using V8 = typename Vec<T>::v8;
  constexpr int D = LPU * 8, UPB = 256 / LPU;
  const long t = blockIdx.x;
  const int tid = threadIdx.x, sub = tid % LPU, d0 = sub * 8;
  const T* row = qkv + t * qkv_stride;
  const int half = rot / 2, hl = half / 8;          // partner lane distance
  const float* cs = rot > 0 ? cos_sin + positions[t] * (long)rot : nullptr;
  const long slot = slot_mapping[t];
  const float qt = query_temperature(xo, positions[t]);
  const int nq = H * maps, nk = G * maps, total = nq + nk;
  for (int u0 = 0; u0 < total; u0 += UPB) {
    const int u = u0 + tid / LPU;
    const bool live = u < total;
    const int uc = live ? u : total - 1;
    const bool is_q = uc < nq;
    const V8 v = ld16<V8>(row + (long)uc * D + d0);
    const float* w = (is_q ? q_w : k_w) + d0;
    float x[8], ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) { x[i] = (float)v[i]; ss += x[i] * x[i]; }
#pragma unroll
    for (int o = LPU / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    const float rs = 1.f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] *= rs * w[i];
    if (rot > 0 && xo.neighbours) {                  // uniform: a pair sits in one lane
      if (d0 < rot) {
        const float* cp = cs + d0 / 2;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float co = cp[i], si = cp[half + i];
          const float a = x[2 * i], b = x[2 * i + 1];
          x[2 * i] = a * co - b * si;
          x[2 * i + 1] = b * co + a * si;
        }
      }
    } else if (rot > 0) {                            // uniform
      const bool lowh = d0 < half, turn = d0 < rot;
      const int partner = (tid & 63) + (lowh ? hl : -hl);
      const float* cp = cs + (lowh ? d0 : d0 - half);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float o = __shfl(x[i], partner & 63, 64);
        if (turn) {
          const float co = cp[i], si = cp[half + i];
          x[i] = lowh ? x[i] * co - o * si : x[i] * co + o * si;
        }
      }
    }
    if (!live) continue;
    T* dst;
    if (is_q) {
      int uo = u;
      if (by_map) {
        const int R = H / G, h = u / maps, mp = u % maps;
        uo = ((h / R) * maps + mp) * R + h % R;
      }
      dst = qn + (t * nq + uo) * (long)D;
    } else {
      if (slot < 0) continue;
      const int uk = u - nq;
      const int g = uk / maps, mp = uk % maps;
      dst = by_map ? k_cache + (((slot / bs) * nk + uk) * (long)bs + slot % bs) * (long)D
                   : k_cache + (((slot / bs) * G + g) * (long)bs + slot % bs) * (long)(maps * D) + (long)mp * D;
    }
    const float mul = is_q ? qt : 1.f;
    V8 o8;
#pragma unroll
    for (int i = 0; i < 8; ++i) o8[i] = (T)(x[i] * mul);
    st16<V8>(dst + d0, o8);
  }
  if (slot >= 0) {
    const T* vsrc = row + (long)total * D;
    T* vdst = v_cache + (slot / bs) * (long)G * Dv * bs + slot % bs;      // [blocks, G, Dv, bs]
    for (int e = tid; e < G * Dv; e += 256) vdst[(long)e * bs] = mixed_value<T>(xo, vsrc[e], t, e);
  }
}

VDA_EXPORT int vda_qk_norm_rope_cache(void* qn, const void* qkv, long qkv_stride, const float* q_w, const float* k_w,
                                      const float* cos_sin, const long* positions, void* k_cache, void* v_cache,
                                      const long* slot_mapping, int T, int H, int G, int D, int Dv, int maps, int rot,
                                      int bs, float eps, int by_map, int neighbours, float q_coef, int q_every,
                                      const void* v_first, long v_first_stride, const float* v_lam, int dtype,
                                      hipStream_t st) {
  if (T <= 0) return 0;
  if (rot < 0 || rot > D || (rot & 1) || maps < 1 || (rot > 0 && !cos_sin) || (v_first && !v_lam)) return -1;
  const QkExtras xo{neighbours, q_coef, q_every, v_first, v_first_stride, v_lam};
  // half-split pairs: the partner sits rot / 16 lanes away; neighbours: inside the lane's own eight values
  const bool vec = (D == 32 || D == 64 || D == 128 || D == 256) && (neighbours ? rot % 8 == 0 : (rot / 2) % 8 == 0) &&
                   qkv_stride % 8 == 0 &&
                   ((uintptr_t)qkv % 32 == 0) && ((uintptr_t)qn % 32 == 0) && ((uintptr_t)k_cache % 32 == 0);
  if (vec) {
#define LV2(TT, LL) hipLaunchKernelGGL((qk_norm_rope_cache_vec_kernel<TT, LL>), dim3(T), dim3(256), 0, st, (TT*)qn,    \
                                       (const TT*)qkv, qkv_stride, q_w, k_w, cos_sin, positions, (TT*)k_cache,          \
                                       (TT*)v_cache, slot_mapping, H, G, Dv, maps, rot, bs, eps, by_map, xo)
#define LV(TT) do { if (D == 32) LV2(TT, 4); else if (D == 64) LV2(TT, 8); else if (D == 128) LV2(TT, 16); else LV2(TT, 32); } while (0)
    if (dtype == VDA_BF16) LV(bf16_t);
    else if (dtype == VDA_F16) LV(f16_t);
    else if (dtype == VDA_F32) LV(float);
    else return -3;
#undef LV
#undef LV2
    VDA_CHECK_LAUNCH();
    return 0;
  }
#define L(TT) hipLaunchKernelGGL((qk_norm_rope_cache_kernel<TT>), dim3(T), dim3(256), 0, st, (TT*)qn, (const TT*)qkv,  \
                                 qkv_stride, q_w, k_w, cos_sin, positions, (TT*)k_cache, (TT*)v_cache, slot_mapping,  \
                                 H, G, D, Dv, maps, rot, bs, eps, by_map, xo)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}

struct MaskedAttnArgs {
  void* out;                 // [T, H * Dv]
  const void* qn;            // [T, H, maps * D]
  const void* k_cache;
  const void* v_cache;
  const int* block_table;
  long bt_stride;
  const int* seq_lens;
  const int* qsl;
  const float* sink;         // [H] or null
  const float* lam;          // one value (maps == 2)
  const void* gate;          // [T, H * Dv] pre-activations or null
  long gate_stride;
  const float* dist_bias;    // [far + 1, H] or null: row min(i - j, far) joins the scores
  int far;
  float scale, eps, out_scale, softcap;
  int window, chunk, maps;
  int H, G, D, Dv, bs;
  int HG;                    // heads per workgroup (of the H / G that share a key / value head)
  int BQ, BK;
};

// first key position the query at position p can see
__device__ __forceinline__ int mask_lower(int p, int window, int chunk) {
  int lo = 0;
  if (window > 0) lo = max(lo, p - window + 1);
  if (chunk > 0) lo = max(lo, p / chunk * chunk);
  return lo;
}

// NACC: output values per thread (M * Dv <= 256 * NACC); M = BQ * heads * maps rows per workgroup (at most 256)
template <typename T, int NACC>
__global__ __launch_bounds__(256) void masked_softmax_attention_kernel(const MaskedAttnArgs a) {
  const int R = a.H / a.G;                      // query heads per key / value head
  const int ngr = (R + a.HG - 1) / a.HG;
  const int g = blockIdx.z / ngr;
  const int hl0 = (blockIdx.z % ngr) * a.HG;    // first of this workgroup's heads inside the group
  const int HN = min(a.HG, R - hl0);
  const int maps = a.maps, D = a.D, Dv = a.Dv, bs = a.bs, BQ = a.BQ, BK = a.BK;
  const int MD = maps * D;
  extern __shared__ float lds[];
  const int Dq = D | 1;                         // odd row pitch: no bank conflicts when lanes walk rows
  const int Kq = MD | 1, Vq = Dv | 1, RS = BK + 1;
  const int M = BQ * HN * maps;                 // row m = (i * HN + hl) * maps + map
  float* qs = lds;                              // [M][Dq]
  float* ks = qs + BQ * a.HG * maps * Dq;       // [BK][Kq]
  float* vs = ks + BK * Kq;                     // [BK][Vq]
  float* sc = vs + BK * Vq;                     // [M][RS] scores, then weights
  float* rm = sc + BQ * a.HG * maps * RS;       // [M] running maximum
  float* rl = rm + BQ * a.HG * maps;            // [M] running sum
  float* ra = rl + BQ * a.HG * maps;            // [M] rescale of this tile

  const int s = blockIdx.y, tid = threadIdx.x;
  const int sl = a.seq_lens[s];
  if (sl <= 0) return;
  const int t0 = a.qsl[s], L = a.qsl[s + 1] - t0;
  const int i0 = blockIdx.x * BQ;
  if (i0 >= L) return;
  const int nq = min(BQ, L - i0);
  const int p0 = sl - L + i0, p1 = p0 + nq;      // positions of the tile's queries: [p0, p1)
  const int* bt = a.block_table + (long)s * a.bt_stride;
  const T* qn = (const T*)a.qn;
  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  const int h0 = g * R + hl0;

  for (int e = tid; e < M * D; e += 256) {
    const int d = e % D, m = e / D;
    const int mp = m % maps, hl = (m / maps) % HN, i = m / (maps * HN);
    qs[m * Dq + d] = i < nq ? (float)qn[((long)(t0 + i0 + i) * a.H + h0 + hl) * MD + mp * D + d] * a.scale : 0.f;
  }
  for (int m = tid; m < M; m += 256) {
    const int hl = (m / maps) % HN;
    if (a.sink) { rm[m] = a.sink[h0 + hl]; rl[m] = 1.f; }       // exp(sink - sink): the sink's share of the sum
    else { rm[m] = -INFINITY; rl[m] = 0.f; }
  }
  float acc[NACC];
#pragma unroll
  for (int n = 0; n < NACC; ++n) acc[n] = 0.f;

  const int lo = mask_lower(p0, a.window, a.chunk);
  const int ntiles = (p1 - lo + BK - 1) / BK;
  for (int tile = 0; tile < ntiles; ++tile) {
    const int j0 = lo + tile * BK;
    const int nk = min(BK, p1 - j0);
    __syncthreads();
    for (int e = tid; e < BK * MD; e += 256) {
      const int d = e % MD, jj = e / MD;
      float v = 0.f;
      if (jj < nk) {
        const int j = j0 + jj;
        v = (float)kc[(((long)bt[j / bs] * a.G + g) * bs + j % bs) * MD + d];
      }
      ks[jj * Kq + d] = v;
    }
    for (int e = tid; e < BK * Dv; e += 256) {
      const int jj = e % BK, d = e / BK;          // consecutive threads walk the keys of one value channel
      float v = 0.f;
      if (jj < nk) {
        const int j = j0 + jj;
        v = (float)vc[(((long)bt[j / bs] * a.G + g) * Dv + d) * bs + j % bs];
      }
      vs[jj * Vq + d] = v;
    }
    __syncthreads();
    for (int e = tid; e < M * BK; e += 256) {
      const int jj = e % BK, m = e / BK;
      const int i = m / (maps * HN);
      const int pi = p0 + i, j = j0 + jj;
      float sv = -INFINITY;
      if (i < nq && jj < nk && j <= pi && j >= mask_lower(pi, a.window, a.chunk)) {
        const float* qp = qs + m * Dq;
        const float* kp = ks + jj * Kq + (m % maps) * D;
        sv = 0.f;
        for (int d = 0; d < D; ++d) sv += qp[d] * kp[d];
        if (a.softcap > 0.f) sv = a.softcap * tanhf(sv / a.softcap);
        if (a.dist_bias) sv += a.dist_bias[(long)min(pi - j, a.far) * a.H + h0 + (m / maps) % HN];
      }
      sc[m * RS + jj] = sv;
    }
    __syncthreads();
    // running maximum and sum per row; scores become weights relative to the new maximum
    for (int m = tid; m < M; m += 256) {
      float* sp = sc + m * RS;
      float mx = rm[m];
      for (int jj = 0; jj < nk; ++jj) mx = fmaxf(mx, sp[jj]);
      const float mu = mx == -INFINITY ? 0.f : mx;
      const float al = expf(rm[m] - mu);        // rm = -inf: 0
      float sum = 0.f;
      for (int jj = 0; jj < nk; ++jj) {
        const float w = expf(sp[jj] - mu);
        sp[jj] = w;
        sum += w;
      }
      rm[m] = mx;
      rl[m] = rl[m] * al + sum;
      ra[m] = al;
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < NACC; ++n) {
      const int e = tid + n * 256;
      if (e < M * Dv) {
        const int d = e % Dv, m = e / Dv;
        const float* wp = sc + m * RS;
        const float* vp = vs + d;
        float v = acc[n] * ra[m];
        for (int jj = 0; jj < nk; ++jj) v += wp[jj] * vp[jj * Vq];
        acc[n] = v;
      }
    }
  }
  __syncthreads();
  // normalised sums through LDS (over the tiles' space), then per (token, head): the maps' combination, its norm,
  // the gate and the store; one wave per (token, head) at a time
  float* oa = lds;                               // [M][Dv]
#pragma unroll
  for (int n = 0; n < NACC; ++n) {
    const int e = tid + n * 256;
    if (e < M * Dv) {
      const float l = rl[e / Dv];
      acc[n] = l > 0.f ? acc[n] / l : 0.f;
    }
  }
  __syncthreads();
#pragma unroll
  for (int n = 0; n < NACC; ++n) {
    const int e = tid + n * 256;
    if (e < M * Dv) oa[e] = acc[n];
  }
  __syncthreads();
  const int lane = tid & 63, wave = tid >> 6;
  const float lam = maps == 2 ? *a.lam : 0.f;
  T* out = (T*)a.out;
  const T* gate = (const T*)a.gate;
  for (int r = wave; r < nq * HN; r += 4) {
    const int hl = r % HN, i = r / HN;
    const float* a1 = oa + (long)(r * maps) * Dv;
    const long tok = t0 + i0 + i;
    const long col = (long)(h0 + hl) * Dv;
    float rsn = 1.f;
    if (maps == 2) {
      float ss = 0.f;
      for (int d = lane; d < Dv; d += 64) {
        const float o = a1[d] - lam * a1[Dv + d];
        ss += o * o;
      }
      ss = wave_sum(ss);
      rsn = a.out_scale / sqrtf(ss / (float)Dv + a.eps);
    }
    for (int d = lane; d < Dv; d += 64) {
      float o = maps == 2 ? (a1[d] - lam * a1[Dv + d]) * rsn : a1[d];
      if (gate) o *= 1.f / (1.f + expf(-(float)gate[tok * a.gate_stride + col + d]));
      out[tok * ((long)a.H * Dv) + col + d] = (T)o;
    }
  }
}

VDA_EXPORT int vda_masked_softmax_attention(void* out, const void* qn, const void* k_cache, const void* v_cache,
                                            const int* block_table, long bt_stride, const int* seq_lens,
                                            const int* qsl, const float* sink, const float* lam, const void* gate,
                                            long gate_stride, float scale, int window, int chunk, int maps, float eps,
                                            float out_scale, int S, int H, int G, int D, int Dv, int bs, int max_q,
                                            float softcap, const float* dist_bias, int far, int dtype,
                                            hipStream_t st) {
  if (S <= 0 || max_q <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0 || maps < 1 || maps > 2 || (maps == 2 && !lam) ||
      (dist_bias && far < 0))
    return -1;
  // tile sizes: the largest query tile (then key tile) whose accumulators fit 64 registers per thread, whose rows
  // fit one workgroup and whose tiles fit 96 KiB of LDS; single decoded tokens take a one-token tile; the heads of
  // a group are dealt to several workgroups when one token's heads alone are too many for that
  const int R = H / G, MD = maps * D;
  const int Dq = D | 1, Kq = MD | 1, Vq = Dv | 1;
  auto lds_of = [&](int bq, int bk, int hg) {
    const size_t M = (size_t)bq * hg * maps;
    const size_t main = M * Dq + (size_t)bk * Kq + (size_t)bk * Vq + M * (bk + 1) + 3 * M;
    const size_t epi = M * Dv;
    return (main > epi ? main : epi) * 4;
  };
  int BQ = 0, BK = 0, HG = R;
  for (; HG >= 1 && !BQ; HG = HG > 1 ? (HG + 1) / 2 : 0) {
    for (int bq = 16; bq >= 1 && !BQ; bq >>= 1) {
      if (bq > 1 && bq / 2 >= max_q) continue;
      const size_t M = (size_t)bq * HG * maps;
      if (M * Dv > 256 * 64 || M > 256) continue;
      for (int bk = 64; bk >= 8; bk >>= 1)
        if (lds_of(bq, bk, HG) <= 96 * 1024) { BQ = bq; BK = bk; break; }
    }
    if (BQ) break;
  }
  if (!BQ) return -2;
  const size_t lds = lds_of(BQ, BK, HG);
  const int per = (BQ * HG * maps * Dv + 255) / 256;
  const int NACC = per <= 8 ? 8 : per <= 16 ? 16 : per <= 32 ? 32 : 64;
  MaskedAttnArgs a;
  a.out = out; a.qn = qn; a.k_cache = k_cache; a.v_cache = v_cache; a.block_table = block_table;
  a.bt_stride = bt_stride; a.seq_lens = seq_lens; a.qsl = qsl; a.sink = sink; a.lam = lam; a.gate = gate;
  a.gate_stride = gate_stride; a.scale = scale; a.eps = eps; a.out_scale = out_scale; a.window = window;
  a.chunk = chunk; a.maps = maps; a.H = H; a.G = G; a.D = D; a.Dv = Dv; a.bs = bs; a.HG = HG; a.BQ = BQ; a.BK = BK;
  a.softcap = softcap; a.dist_bias = dist_bias; a.far = far;
  dim3 grid((max_q + BQ - 1) / BQ, S, G * ((R + HG - 1) / HG)), block(256);
#define L2(TT, NA)                                                                                                  \
  do {                                                                                                              \
    if (lds > 48 * 1024) {                                                                                          \
      hipError_t e = hipFuncSetAttribute((const void*)masked_softmax_attention_kernel<TT, NA>,                      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                     \
      if (e != hipSuccess) return (int)e;                                                                           \
    }                                                                                                               \
    hipLaunchKernelGGL((masked_softmax_attention_kernel<TT, NA>), grid, block, lds, st, a);                         \
  } while (0)
#define L(TT)                                                                                                       \
  do {                                                                                                              \
    if (NACC == 8) L2(TT, 8); else if (NACC == 16) L2(TT, 16); else if (NACC == 32) L2(TT, 32); else L2(TT, 64);    \
  } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
  VDA_CHECK_LAUNCH();
  return 0;
}

// a [T, G, maps, R, Dv] (the matrix-core kernels' output with one query row per map) -> out [T, H * Dv]:
// o = a1 - lam * a2 divided by its root mean square over Dv and scaled (maps == 2), times sigmoid(gate).
// One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(256) void map_combine_kernel(T* __restrict__ out, const T* __restrict__ a,
                                                          const float* __restrict__ lam_p, const T* __restrict__ gate,
                                                          long gate_stride, long n_rows, int H, int G, int Dv,
                                                          int maps, float eps, float out_scale) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  const int lane = threadIdx.x & 63;
  const long t = row / H;
  const int h = (int)(row % H), R = H / G;
  const T* a1 = a + ((t * G + h / R) * maps * R + h % R) * (long)Dv;
  const T* a2 = a1 + (long)R * Dv;
  const float lam = maps == 2 ? *lam_p : 0.f;
  float rsn = 1.f;
  if (maps == 2) {
    float ss = 0.f;
    for (int d = lane; d < Dv; d += 64) {
      const float o = (float)a1[d] - lam * (float)a2[d];
      ss += o * o;
    }
    ss = wave_sum(ss);
    rsn = out_scale / sqrtf(ss / (float)Dv + eps);
  }
  for (int d = lane; d < Dv; d += 64) {
    float o = maps == 2 ? ((float)a1[d] - lam * (float)a2[d]) * rsn : (float)a1[d];
    if (gate) o *= 1.f / (1.f + expf(-(float)gate[t * gate_stride + (long)h * Dv + d]));
    out[row * Dv + d] = (T)o;
  }
}

VDA_EXPORT int vda_map_combine(void* out, const void* a, const float* lam, const void* gate, long gate_stride, int T,
                               int H, int G, int Dv, int maps, float eps, float out_scale, int dtype, hipStream_t st) {
  if (T <= 0) return 0;
  if (H % G || maps < 1 || maps > 2 || (maps == 2 && !lam)) return -1;
  const long rows = (long)T * H;
#define L(TT) hipLaunchKernelGGL((map_combine_kernel<TT>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st,         \
                                 (TT*)out, (const TT*)a, lam, (const TT*)gate, gate_stride, rows, H, G, Dv, maps, eps, \
                                 out_scale)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}
