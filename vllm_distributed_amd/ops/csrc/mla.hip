// Multi-head latent attention (DeepSeek-V2 / V3) over a latent KV cache.
//
// Per token the cache holds ONE latent row instead of per-head keys and values:
//   kc [num_blocks, BS, DK]   DK = kv_lora_rank + rope_dim: the normalised latent c_kv followed by
//                             the rotated shared key k_pe (what the query side dots against)
//   vt [num_blocks, DV, BS]   DV = kv_lora_rank: the same latent, transposed, so that the P.V MFMA
//                             reads 8 consecutive keys of one latent dimension with one 16-byte load
// With the key up-projection absorbed into the query (q_abs = q_nope . W_UK) and the value
// up-projection applied after attention (o = o_lat . W_UV), every head attends over the same latent
// rows: multi-query attention with head sizes DK / DV.  The cache is (DK + DV) elements per token,
// against 2 * heads * head_dim for expanded heads (57x smaller for DeepSeek-V3).  With an fp8 cache both copies
// hold e4m3 bytes of value / kv_scale (one scale for the latent and the rotated key): half the bytes again; the
// kernel widens them on the way into the MFMA operands and folds the scale into the logits and the output
// (reference: csrc/cache_kernels.cu:309-343 concat_and_cache_mla with kv_cache_dtype fp8).
//
// Kernel: the MFMA scheme of attention.hip (S^T = K.Q^T with keys on the MFMA row, O^T += V^T.P^T),
// 16 (token, head) query columns per workgroup, the 4 waves split the keys and merge through LDS;
// grid.z splits long contexts further (partials + reduce).  One code path serves decode and
// (chunked) prefill; per-column causal limits come from the token index.
// Role of the reference's csrc/cache_kernels.cu::concat_and_cache_mla and its MLA decode backends
// (vllm/v1/attention/backends/mla/*, vllm/attention/ops/triton_decode_attention.py).
#include "common.h"

// 2^x as the bare v_exp_f32 instruction (fexp2() adds a range check and rescale for sub-normal results)
__device__ __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- cache write -----------------------------------------------------------------------------------
template <typename T, bool F8>
__global__ __launch_bounds__(256) void mla_cache_write_kernel(const T* __restrict__ kv_c, const T* __restrict__ k_pe,
                                                              typename KVElem<T, F8>::type* __restrict__ kc,
                                                              typename KVElem<T, F8>::type* __restrict__ vt,
                                                              const long* __restrict__ slot_mapping, int R, int ROPE,
                                                              int BS, long c_stride, long pe_stride, float inv_scale) {
  using CT = typename KVElem<T, F8>::type;
  const int t = blockIdx.x;
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  const long blk = slot / BS;
  const int off = (int)(slot % BS);
  const int DK = R + ROPE;
  CT* krow = kc + (blk * BS + off) * (long)DK;
  for (int d = threadIdx.x; d < DK; d += 256) {
    if (d < R) {
      const T v = kv_c[(long)t * c_stride + d];
      KVStore<T, F8>::st1(krow + d, v, inv_scale);
      KVStore<T, F8>::st1(vt + (blk * R + d) * (long)BS + off, v, inv_scale);
    } else {
      KVStore<T, F8>::st1(krow + d, k_pe[(long)t * pe_stride + (d - R)], inv_scale);
    }
  }
}

// kv_fp8: the cache holds e4m3 bytes of value / kv_scale
VDA_EXPORT int vda_mla_cache_write(const void* kv_c, const void* k_pe, void* kc, void* vt, const long* slot_mapping,
                                   int T, int R, int ROPE, int BS, long c_stride, long pe_stride, int dtype,
                                   int kv_fp8, float kv_scale, hipStream_t st) {
  if (T <= 0) return 0;
  dim3 grid(T), block(256);
  const float inv = kv_fp8 ? 1.f / kv_scale : 1.f;
#define W(TT, F8)                                                                                                   \
  hipLaunchKernelGGL((mla_cache_write_kernel<TT, F8>), grid, block, 0, st, (const TT*)kv_c, (const TT*)k_pe,          \
                     (typename KVElem<TT, F8>::type*)kc, (typename KVElem<TT, F8>::type*)vt, slot_mapping, R, ROPE, BS, \
                     c_stride, pe_stride, inv)
  if (dtype == VDA_BF16) { if (kv_fp8) W(bf16_t, true); else W(bf16_t, false); }
  else if (dtype == VDA_F16) { if (kv_fp8) W(f16_t, true); else W(f16_t, false); }
  else return -3;
#undef W
  VDA_CHECK_LAUNCH();
  return 0;
}

// ---- attention ---------------------------------------------------------------------------------------
struct MlaParams {
  const void* q;            // [T, H, DK]: absorbed q_nope followed by rotated q_pe
  const void* kc;
  const void* vt;
  void* out;                // [T, H, DV] latent-space output
  float* part_out;          // [T, H, nsplit, DV]
  float* part_lse;          // [T, H, nsplit] (log2 domain)
  const int* block_table;
  const int* seq_lens;
  const int* q_start_loc;
  int H, BS, max_blocks, nsplit;
  long q_stride, out_stride;
  float scale;              // softmax scale, times the cache scale for an fp8 cache
  float v_scale;            // 1, or the cache scale for an fp8 cache
  int window;               // > 0: a query at position i sees the keys j with 0 <= i - j < window
  const float* sink;        // [H] or null: exp(sink[h]) joins head h's softmax denominator, with no key and no value
  int wave_cols;            // 1: every wave takes 16 columns of its own over all keys (prompts: neighbouring tokens
                            //    walk the same keys at the same time, so the rows come from the cache near the CU);
                            // 0: the 4 waves share 16 columns and split the keys (few query tokens)
};

template <typename T, int DK, int DV, bool F8>
__global__ __launch_bounds__(256) void mla_attention_kernel(MlaParams p) {
  using V8 = typename Vec<T>::v8;
  using V4 = typename Vec<T>::v4;
  using CT = typename KVElem<T, F8>::type;
  constexpr int KS = DK / 32;        // MFMA k-steps over the query/key width
  constexpr int NT = DV / 16;        // 16-row tiles of the latent output
  constexpr int DQ = DK / 4;         // key dims owned by one lane group
  constexpr int VCH = NT >= 8 ? 8 : NT;   // V tiles in flight at once (register budget)
  static_assert(DK % 32 == 0 && DV % 16 == 0 && DQ % 8 == 0 && NT % VCH == 0, "unsupported latent sizes");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int seq = blockIdx.x;
  const int qs = p.q_start_loc[seq];
  const int q_len = p.q_start_loc[seq + 1] - qs;
  const int seq_len = p.seq_lens[seq];
  // first (token, head) column of this workgroup, or of this wave
  const int c0 = p.wave_cols ? (blockIdx.y * 4 + wave) * 16 : blockIdx.y * 16;
  if (seq_len <= 0 || c0 >= q_len * p.H) return;       // wave_cols: no barrier follows, waves may leave alone
  const int ctx = seq_len - q_len;
  const int BS = p.BS;
  const int* bt = p.block_table + (long)seq * p.max_blocks;
  const int nblk_valid = (seq_len + BS - 1) / BS;

  // this lane's query column
  const int c = c0 + r;
  const int ti = c / p.H, head = c % p.H;
  const bool valid = ti < q_len;
  const int limit = valid ? ctx + ti + 1 : 0;
  V8 qf[KS];
  {
    const T* qp = (const T*)p.q + (long)(qs + (valid ? ti : 0)) * p.q_stride + (long)head * DK + g * DQ;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = valid ? ld16<V8>(qp + 8 * s) : V8{};
  }
  const int first = p.window > 0 ? max(limit - p.window, 0) : 0;      // first visible key of this column
  int hi = limit, lo = valid ? first : 0x7fffffff;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    hi = max(hi, __shfl_xor(hi, o, 64));
    lo = min(lo, __shfl_xor(lo, o, 64));
  }
  // key steps of 32 (those before every column's window are never loaded): partition over grid.z, then deal to
  // the 4 waves
  int step_hi = (hi + 31) / 32;
  const int step_lo = min(lo / 32, step_hi);
  const int per = (step_hi - step_lo + p.nsplit - 1) / p.nsplit;
  const int a0 = step_lo + blockIdx.z * per;
  step_hi = min(step_hi, a0 + per);

  // a sink is a score without key or value: the running maximum starts there and the sum with its weight of one,
  // in one lane group, one wave and one key partition, so that it counts once
  const bool own_sink = p.sink && valid && blockIdx.z == 0 && (p.wave_cols || wave == 0);
  float m = own_sink ? p.sink[head] * 1.4426950408889634f : -INFINITY, l = (own_sink && g == 0) ? 1.f : 0.f;
  f32x4 acc[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) acc[n] = f32x4{0, 0, 0, 0};
  const CT* kc = (const CT*)p.kc;
  const CT* vt = (const CT*)p.vt;
  const int krow0 = 8 * (r >> 2) + (r & 3);     // tile u, row r <-> key 8*(r>>2) + 4u + (r&3) of the step
  const float sc = p.scale * 1.4426950408889634f;

  for (int step = p.wave_cols ? a0 : a0 + wave; step < step_hi; step += p.wave_cols ? 1 : 4) {
    const int tb = step * 32 + 8 * g;            // first of this lane's 8 keys
    f32x4 s2[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int tok = step * 32 + krow0 + 4 * u;
      const int bi = max(min(tok / BS, nblk_valid - 1), 0);
      const CT* kp = kc + ((long)bt[bi] * BS + (tok % BS)) * DK + g * DQ;
      f32x4 s = {0, 0, 0, 0};
#pragma unroll
      for (int k = 0; k < KS; ++k) s = mfma16(KVLoad<T, F8>::ld(kp + 8 * k), qf[k], s);
      s2[u] = s;
    }
    float sv[8] = {s2[0][0], s2[0][1], s2[0][2], s2[0][3], s2[1][0], s2[1][1], s2[1][2], s2[1][3]};
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      sv[j] = (tb + j < limit && tb + j >= first) ? sv[j] * sc : -INFINITY;
      mx = fmaxf(mx, sv[j]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fexp2(m - m_use);
    m = m_new;
    float ps = 0.f;
    V8 pb;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float e = fexp2(sv[j] - m_use);
      ps += e;
      pb[j] = (T)e;
    }
    l = l * alpha + ps;
    const int bi = max(min(tb / BS, nblk_valid - 1), 0);
    const CT* vp = vt + ((long)bt[bi] * DV + r) * BS + (tb % BS);
#pragma unroll
    for (int n0 = 0; n0 < NT; n0 += VCH) {
      V8 vf[VCH];
#pragma unroll
      for (int n = 0; n < VCH; ++n) vf[n] = KVLoad<T, F8>::ld(vp + (long)(n0 + n) * 16 * BS);
#pragma unroll
      for (int n = 0; n < VCH; ++n) {
        acc[n0 + n] *= alpha;
        acc[n0 + n] = mfma16(vf[n], pb, acc[n0 + n]);
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);

  // ---- merge the 4 waves into wave 0, one sender at a time (one staging buffer keeps LDS at NT KB) ----
  __shared__ f32x4 s_acc[NT][64];
  __shared__ float s_ml[2][64];
  for (int snd = 1; snd < 4 && !p.wave_cols; ++snd) {
    if (wave == snd) {
      s_ml[0][lane] = m;
      s_ml[1][lane] = l;
#pragma unroll
      for (int n = 0; n < NT; ++n) s_acc[n][lane] = acc[n];
    }
    __syncthreads();
    if (wave == 0) {
      const float m2 = s_ml[0][lane], l2 = s_ml[1][lane];
      const float M = fmaxf(m, m2);
      const float Mu = (M == -INFINITY) ? 0.f : M;
      const float f1 = fexp2(m - Mu), f2 = fexp2(m2 - Mu);
      l = l * f1 + l2 * f2;
      m = M;
#pragma unroll
      for (int n = 0; n < NT; ++n) acc[n] = acc[n] * f1 + s_acc[n][lane] * f2;
    }
    __syncthreads();
  }
  if ((wave != 0 && !p.wave_cols) || !valid) return;
  const float inv = l > 0.f ? p.v_scale / l : 0.f;
  const long tok = qs + ti;
  if (p.nsplit == 1) {
    T* op = (T*)p.out + tok * p.out_stride + (long)head * DV + 4 * g;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      V4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (T)(acc[n][i] * inv);
      *reinterpret_cast<V4*>(op + 16 * n) = o;
    }
  } else {
    const long pi = (tok * p.H + head) * p.nsplit + blockIdx.z;
    float* po = p.part_out + pi * DV + 4 * g;
#pragma unroll
    for (int n = 0; n < NT; ++n) *reinterpret_cast<f32x4*>(po + 16 * n) = acc[n] * inv;
    if (g == 0) {
      const float Mu = (m == -INFINITY) ? 0.f : m;
      p.part_lse[pi] = l > 0.f ? Mu + log2f(l) : -INFINITY;
    }
  }
}

// ---- prompts: key / value tiles staged in LDS for four column groups ---------------------------------------------
// One workgroup = 64 consecutive (token, head) columns of one sequence, 16 per wave.  Every 32-key step is copied
// from the cache into LDS once (the latent rows in the order the MFMA row tiles want them, the transposed latent as
// it lies) and read from there by all four waves: a quarter of the cache traffic of the form above, and the A
// operands come from LDS instead of waiting on the cache one MFMA at a time.  Everything else -- operand layouts,
// online softmax, masks -- is the form above; a wave skips the steps outside its own columns' range.
template <typename T, int DK, int DV>
__global__ __launch_bounds__(256) void mla_prefill_kernel(MlaParams p) {
  using V8 = typename Vec<T>::v8;
  using V4 = typename Vec<T>::v4;
  constexpr int KS = DK / 32, NT = DV / 16, DQ = DK / 4;
  constexpr int KROW = DK + 8;       // padded LDS rows: consecutive rows fall into different 16-byte bank groups
  constexpr int VROW = 32 + 8;
  static_assert(DK % 32 == 0 && DV % 16 == 0 && DQ % 8 == 0, "unsupported latent sizes");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* ks = reinterpret_cast<T*>(smem);                 // [32][KROW]: row u * 16 + r holds key 8 (r >> 2) + 4 u + (r & 3)
  T* vs = ks + 32 * KROW;                             // [DV][VROW]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int seq = blockIdx.x;
  const int qs = p.q_start_loc[seq];
  const int q_len = p.q_start_loc[seq + 1] - qs;
  const int seq_len = p.seq_lens[seq];
  const int cw = blockIdx.y * 64;                    // first column of the workgroup
  if (seq_len <= 0 || cw >= q_len * p.H) return;     // the whole workgroup leaves
  const int ctx = seq_len - q_len;
  const int BS = p.BS;
  const int* bt = p.block_table + (long)seq * p.max_blocks;
  const int nblk_valid = (seq_len + BS - 1) / BS;

  // this lane's query column
  const int c = cw + wave * 16 + r;
  const int ti = c / p.H, head = c % p.H;
  const bool valid = ti < q_len;
  const int limit = valid ? ctx + ti + 1 : 0;
  const int first = p.window > 0 ? max(limit - p.window, 0) : 0;
  V8 qf[KS];
  {
    const T* qp = (const T*)p.q + (long)(qs + (valid ? ti : 0)) * p.q_stride + (long)head * DK + g * DQ;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = valid ? ld16<V8>(qp + 8 * s) : V8{};
  }
  int hi = limit, lo = valid ? first : 0x7fffffff;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    hi = max(hi, __shfl_xor(hi, o, 64));
    lo = min(lo, __shfl_xor(lo, o, 64));
  }
  const int my_hi = (hi + 31) / 32, my_lo = min(lo / 32, my_hi);      // this wave's steps
  // the workgroup's steps, from its first and last token (the same in every wave)
  const int t_first = cw / p.H, t_last = min((cw + 63) / p.H, q_len - 1);
  const int wg_hi = (ctx + t_last + 1 + 31) / 32;
  const int wg_lo = p.window > 0 ? max(ctx + t_first + 1 - p.window, 0) / 32 : 0;

  const bool own_sink = p.sink && valid;               // see mla_attention_kernel
  float m = own_sink ? p.sink[head] * 1.4426950408889634f : -INFINITY, l = (own_sink && g == 0) ? 1.f : 0.f;
  f32x4 acc[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) acc[n] = f32x4{0, 0, 0, 0};
  const T* kc = (const T*)p.kc;
  const T* vt = (const T*)p.vt;
  const float sc = p.scale * 1.4426950408889634f;

  for (int step = wg_lo; step < wg_hi; ++step) {
    __syncthreads();                                   // the tiles of the step before are read
    // the pages this step touches, looked up once (the same for every lane); a thread copies pieces of ONE latent
    // row (8 threads per row) and of ONE 8-key column of the transposed tile, so that pages and row addresses are
    // worked out once per step; all loads of a tile are in flight together before the first store to LDS
    const int b0 = step * 32 / BS;
    int pg[5];
#pragma unroll
    for (int j = 0; j < 5; ++j) pg[j] = bt[max(min(b0 + j, nblk_valid - 1), 0)];
    auto page = [&](int tok) {
      const int j = tok / BS - b0;
      return j == 0 ? pg[0] : j == 1 ? pg[1] : j == 2 ? pg[2] : j == 3 ? pg[3] : pg[4];
    };
    {
      constexpr int CH = DK / 8, KI = (CH + 7) / 8;      // 16-byte pieces per row; pieces per thread
      const int L = tid >> 3, c0 = tid & 7;
      const int rr = L & 15, u = L >> 4;
      const int tok = step * 32 + 8 * (rr >> 2) + 4 * u + (rr & 3);
      const T* src = kc + ((long)page(tok) * BS + (tok % BS)) * DK + c0 * 8;
      T* dst = ks + L * KROW + c0 * 8;
      V8 tmp[KI];
#pragma unroll
      for (int i = 0; i < KI; ++i)
        if (c0 + 8 * i < CH) tmp[i] = ld16<V8>(src + 64 * i);
#pragma unroll
      for (int i = 0; i < KI; ++i)
        if (c0 + 8 * i < CH) st16<V8>(dst + 64 * i, tmp[i]);
    }
    {
      constexpr int VI = (DV + 63) / 64;                 // rows per thread
      const int ch = tid & 3, d0 = tid >> 2;
      const int tok = step * 32 + 8 * ch;
      const T* src = vt + ((long)page(tok) * DV + d0) * BS + (tok % BS);
      T* dst = vs + d0 * VROW + ch * 8;
      V8 tmp[VI];
#pragma unroll
      for (int i = 0; i < VI; ++i)
        if (d0 + 64 * i < DV) tmp[i] = ld16<V8>(src + (long)64 * i * BS);
#pragma unroll
      for (int i = 0; i < VI; ++i)
        if (d0 + 64 * i < DV) st16<V8>(dst + 64 * i * VROW, tmp[i]);
    }
    __syncthreads();
    if (step < my_lo || step >= my_hi) continue;       // wave-uniform
    const int tb = step * 32 + 8 * g;                  // first of this lane's 8 keys
    f32x4 s2[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const T* kp = ks + (u * 16 + r) * KROW + g * DQ;
      f32x4 s = {0, 0, 0, 0};
#pragma unroll
      for (int k = 0; k < KS; ++k) s = mfma16(ld16<V8>(kp + 8 * k), qf[k], s);
      s2[u] = s;
    }
    float sv[8] = {s2[0][0], s2[0][1], s2[0][2], s2[0][3], s2[1][0], s2[1][1], s2[1][2], s2[1][3]};
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      sv[j] = (tb + j < limit && tb + j >= first) ? sv[j] * sc : -INFINITY;
      mx = fmaxf(mx, sv[j]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = (m == -INFINITY) ? 1.f : fexp2(m - m_use);     // nothing summed yet: nothing to rescale
    m = m_new;
    float ps = 0.f;
    V8 pb;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float e = fexp2(sv[j] - m_use);
      ps += e;
      pb[j] = (T)e;
    }
    l = l * alpha + ps;
    const T* vp = vs + r * VROW + 8 * g;
    if (__any(alpha != 1.f)) {                          // the running maximum moved in some column: rescale (rare
#pragma unroll                                          //  after a column's first steps)
      for (int n = 0; n < NT; ++n) acc[n] *= alpha;
    }
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[n] = mfma16(ld16<V8>(vp + n * 16 * VROW), pb, acc[n]);
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!valid) return;
  const float inv = l > 0.f ? p.v_scale / l : 0.f;
  T* op = (T*)p.out + (long)(qs + ti) * p.out_stride + (long)head * DV + 4 * g;
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    V4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (T)(acc[n][i] * inv);
    *reinterpret_cast<V4*>(op + 16 * n) = o;
  }
}

// merge split partials: one wave per (token, head)
template <typename T, int DV>
__global__ __launch_bounds__(64) void mla_reduce_kernel(T* out, const float* part_out, const float* part_lse, int H,
                                                        int nsplit, long out_stride) {
  const long th = blockIdx.x;
  const int lane = threadIdx.x;
  // lane s holds partition s (nsplit <= 64): wave reductions for the maximum and the weight sum, weights
  // handed out by shuffles, partitions without keys skipped
  const float mine = lane < nsplit ? part_lse[th * nsplit + lane] : -INFINITY;
  float M = mine;
#pragma unroll
  for (int o_ = 32; o_ > 0; o_ >>= 1) M = fmaxf(M, __shfl_xor(M, o_, 64));
  const float Mu = (M == -INFINITY) ? 0.f : M;
  const float w_mine = (mine == -INFINITY) ? 0.f : fexp2(mine - Mu);
  float W = w_mine;
#pragma unroll
  for (int o_ = 32; o_ > 0; o_ >>= 1) W += __shfl_xor(W, o_, 64);
  constexpr int PER = (DV + 63) / 64;
  float o[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) o[i] = 0.f;
#pragma unroll 2
  for (int s = 0; s < nsplit; ++s) {
    const float w = __shfl(w_mine, s, 64);
    if (w == 0.f) continue;
    const float* po = part_out + (th * nsplit + s) * DV;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int d = lane + 64 * i;
      if (d < DV) o[i] += w * po[d];
    }
  }
  const float inv = W > 0.f ? 1.f / W : 0.f;
  const long tok = th / H, head = th % H;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int d = lane + 64 * i;
    if (d < DV) out[tok * out_stride + head * DV + d] = (T)(o[i] * inv);
  }
}

template <typename T, int DK, int DV>
static int launch_mla(const MlaParams& p, int S, int T_tokens, int max_q, bool f8, hipStream_t st) {
  dim3 block(256), grid(S, p.wave_cols ? (max_q * p.H + 63) / 64 : (max_q * p.H + 15) / 16, p.nsplit);
  if (p.wave_cols && !f8) {
    // prompts on a 16-bit cache: the LDS-staged form
    constexpr int lds = (32 * (DK + 8) + DV * 40) * (int)sizeof(T);
    static bool ready = false;          // one attribute call per instantiation
    if (!ready && lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute((const void*)mla_prefill_kernel<T, DK, DV>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      if (e != hipSuccess) return (int)e;
      ready = true;
    }
    hipLaunchKernelGGL((mla_prefill_kernel<T, DK, DV>), grid, block, lds, st, p);
    return 0;
  }
  if (f8) hipLaunchKernelGGL((mla_attention_kernel<T, DK, DV, true>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((mla_attention_kernel<T, DK, DV, false>), grid, block, 0, st, p);
  if (p.nsplit > 1)
    hipLaunchKernelGGL((mla_reduce_kernel<T, DV>), dim3((unsigned)((long)T_tokens * p.H)), dim3(64), 0, st,
                       (T*)p.out, p.part_out, p.part_lse, p.H, p.nsplit, p.out_stride);
  return 0;
}

VDA_EXPORT int vda_mla_supported(int DK, int DV) {
  return (DK == 576 && DV == 512) || (DK == 96 && DV == 64) || (DK == 160 && DV == 128);
}

VDA_EXPORT int vda_mla_attention(void* out, const void* q, const void* kc, const void* vt, const int* block_table,
                                 const int* seq_lens, const int* q_start_loc, float* part_out, float* part_lse,
                                 int S, int T_tokens, int H, int DK, int DV, int BS, int max_blocks, int nsplit,
                                 int max_q, long q_stride, long out_stride, float scale, int dtype, int kv_fp8,
                                 float kv_scale, int window, const float* sink, hipStream_t st) {
  if (S <= 0 || T_tokens <= 0) return 0;
  if (!vda_mla_supported(DK, DV) || BS % 8 || nsplit < 1 || nsplit > 64 || (nsplit > 1 && (!part_out || !part_lse)))
    return -1;      // (the reduce kernel keeps one partition per lane)
  MlaParams p;
  p.q = q; p.kc = kc; p.vt = vt; p.out = out; p.part_out = part_out; p.part_lse = part_lse;
  p.block_table = block_table; p.seq_lens = seq_lens; p.q_start_loc = q_start_loc;
  p.H = H; p.BS = BS; p.max_blocks = max_blocks; p.nsplit = nsplit;
  p.q_stride = q_stride; p.out_stride = out_stride;
  p.scale = scale * (kv_fp8 ? kv_scale : 1.f); p.v_scale = kv_fp8 ? kv_scale : 1.f;
  p.window = window > 0 ? window : 0;
  p.sink = sink;
  p.wave_cols = (nsplit == 1 && (long)max_q * H >= 64) ? 1 : 0;
  const bool f8 = kv_fp8 != 0;
  int rc = 0;
#define BYD(TT) do { if (DK == 576) rc = launch_mla<TT, 576, 512>(p, S, T_tokens, max_q, f8, st);      \
                     else if (DK == 96) rc = launch_mla<TT, 96, 64>(p, S, T_tokens, max_q, f8, st);    \
                     else rc = launch_mla<TT, 160, 128>(p, S, T_tokens, max_q, f8, st); } while (0)
  if (dtype == VDA_BF16) BYD(bf16_t);
  else if (dtype == VDA_F16) BYD(f16_t);
  else return -3;
#undef BYD
  if (rc) return rc;
  VDA_CHECK_LAUNCH();
  return 0;
}
