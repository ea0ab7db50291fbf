// What lies between a mixer's first projection and its attention, and between its attention (or
// recurrence) and its output projection, for mixers whose queries and keys are normed:
//
// ptl_qkv_prepare: one workgroup a token, or several that share its heads when the tokens are few.
//   Reads the float32 row of the projection (q | k | v at
//   given columns), adds the biases, norms queries and keys (RMS norm over every head on its own
//   with one weight for all heads, or over the whole of q and the whole of k with a weight of that
//   size, or not at all), turns the first rot_dims entries of every head by the token's position
//   (entry i with entry i + rot_dims / 2; sine and cosine times ``mag``), writes the queries
//   [T, Hq, Dk] in the engine's type and the keys and values into the token's cache slot
//   (k_cache [pages, Hk, page_size, Dk], v_cache [pages, Hv, page_size, Dv]). A layer that reads
//   another's keys and values has none of its own: k_off < 0.
//
// ptl_head_norm_gate: one wave a (token, head). From float32 results a [T, HA, Dv]:
//   o = a[h * maps] - lam * a[h * maps + 1] (maps 2) or a[h] (maps 1); o / sqrt(mean(o^2) + eps)
//   over the head's Dv values, times a weight (one for all heads, or one a head, or none), times a
//   constant, times act(gate) with the gate read from a float32 matrix at given columns
//   (sigmoid, SiLU, or none). The result [T, H * Dv] is in the engine's type.
//
// All arithmetic is float32: the angle is float(position) * frequency, sinf / cosf / expf are the
// accurate ones.
#include "common.h"
#include <math.h>

#define NORM_NONE 0
#define NORM_HEAD 1
#define NORM_WHOLE 2

// A token's work is cut into ``gridDim.y`` slices of whole heads (queries, then keys, then values),
// so that the few tokens of a decode step still fill the chip. Every slice reads the whole row of
// q and k when the norm is over the whole of them, else only its heads.
template <typename TO>
__global__ void __launch_bounds__(256)
qkv_prepare_kernel(TO* __restrict__ q_out, const float* __restrict__ p, long ldp, int q_off, int k_off,
                   int v_off, const float* __restrict__ qb, const float* __restrict__ kb,
                   const float* __restrict__ vb, int norm_mode, const float* __restrict__ qw,
                   const float* __restrict__ kw, float eps, int rot_dims,
                   const float* __restrict__ inv_freq, float mag, const int32_t* __restrict__ positions,
                   const int32_t* __restrict__ slots, TO* __restrict__ k_cache, TO* __restrict__ v_cache,
                   int Hq, int Hk, int Hv, int Dk, int Dv, int page_size, int heads_per_slice) {
  extern __shared__ float lds[];
  const bool own = k_off >= 0;
  const int nq = Hq * Dk, nk = own ? Hk * Dk : 0;
  const int heads_qk = Hq + (own ? Hk : 0);
  float* raw = lds;                       // [nq + nk]: q then k, bias added (this slice's heads, or all)
  float* rs = raw + nq + nk;              // [Hq + Hk] (per head) or [2] (whole): 1 / rms
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  // this slice: heads h_lo .. h_hi of q | k | v counted in one row
  const int h_lo = blockIdx.y * heads_per_slice;
  const int h_hi = min(h_lo + heads_per_slice, heads_qk + (own ? Hv : 0));
  const int qk_lo = min(h_lo, heads_qk), qk_hi = min(h_hi, heads_qk);      // its q and k heads
  const float* row = p + (size_t)t * ldp;
  if (qk_lo < qk_hi) {
    const int e_lo = norm_mode == NORM_WHOLE ? 0 : qk_lo * Dk;
    const int e_hi = norm_mode == NORM_WHOLE ? nq + nk : qk_hi * Dk;
    for (int e = e_lo + tid; e < e_hi; e += 256)
      raw[e] = e < nq ? row[q_off + e] + (qb ? qb[e] : 0.f) : row[k_off + e - nq] + (kb ? kb[e - nq] : 0.f);
    __syncthreads();
    if (norm_mode == NORM_HEAD) {
      const int wave = tid >> 6, lane = tid & 63;
      for (int h = qk_lo + wave; h < qk_hi; h += 4) {
        const float* x = raw + (size_t)h * Dk;          // (k heads follow the q heads, same size)
        float ss = 0.f;
        for (int d = lane; d < Dk; d += 64) ss = fmaf(x[d], x[d], ss);
        ss = wave_sum(ss);
        if (lane == 0) rs[h] = 1.0f / sqrtf(ss / (float)Dk + eps);
      }
      __syncthreads();
    } else if (norm_mode == NORM_WHOLE) {
      float ss = 0.f;
      for (int e = tid; e < nq; e += 256) ss = fmaf(raw[e], raw[e], ss);
      ss = block_sum(ss, scratch);
      float sk = 0.f;
      for (int e = tid; e < nk; e += 256) sk = fmaf(raw[nq + e], raw[nq + e], sk);
      sk = block_sum(sk, scratch);
      if (tid == 0) {
        rs[0] = 1.0f / sqrtf(ss / (float)nq + eps);
        rs[1] = nk ? 1.0f / sqrtf(sk / (float)nk + eps) : 0.f;
      }
      __syncthreads();
    }
  }
  const int half = rot_dims >> 1;
  const float pos = (float)positions[t];
  const int slot = slots ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, in_page = slot >= 0 ? slot % page_size : 0;
  for (int e = qk_lo * Dk + tid; e < qk_hi * Dk; e += 256) {
    const bool is_k = e >= nq;
    const int i = is_k ? e - nq : e;                  // index inside q or inside k
    const int h = i / Dk, d = i - h * Dk;
    const float* w = is_k ? kw : qw;
    float r = 1.f;
    if (norm_mode == NORM_HEAD) r = rs[is_k ? Hq + h : h];
    else if (norm_mode == NORM_WHOLE) r = rs[is_k ? 1 : 0];
    const int wi = norm_mode == NORM_WHOLE ? i : d;
    float val = raw[e] * r;
    if (norm_mode != NORM_NONE) val *= w[wi];
    if (d < rot_dims) {
      const int dp = d < half ? d + half : d - half;
      float other = raw[e + dp - d] * r;
      if (norm_mode != NORM_NONE) other *= w[wi + dp - d];
      const float a = pos * inv_freq[d < half ? d : d - half];
      const float c = cosf(a) * mag, s = sinf(a) * mag;
      val = d < half ? val * c - other * s : val * c + other * s;
    }
    if (!is_k) {
      q_out[(size_t)t * nq + i] = from_float<TO>(val);
    } else if (slot >= 0) {
      k_cache[(((size_t)page * Hk + h) * page_size + in_page) * Dk + d] = from_float<TO>(val);
    }
  }
  if (own && slot >= 0 && h_hi > heads_qk) {
    const int v_lo = max(h_lo, heads_qk) - heads_qk, v_hi = h_hi - heads_qk;
    for (int e = v_lo * Dv + tid; e < v_hi * Dv; e += 256) {
      const int h = e / Dv, d = e - h * Dv;
      v_cache[(((size_t)page * Hv + h) * page_size + in_page) * Dv + d] =
          from_float<TO>(row[v_off + e] + (vb ? vb[e] : 0.f));
    }
  }
}

extern "C" int ptl_qkv_prepare(void* q_out, const float* p, long ldp, int q_off, int k_off, int v_off,
                               const float* qb, const float* kb, const float* vb, int norm_mode,
                               const float* qw, const float* kw, float eps, int rot_dims,
                               const float* inv_freq, float mag, const int32_t* positions,
                               const int32_t* slots, void* k_cache, void* v_cache, int T_, int Hq, int Hk,
                               int Hv, int Dk, int Dv, int page_size, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (Hq <= 0 || Dk <= 0 || rot_dims < 0 || rot_dims > Dk || (rot_dims & 1) || (rot_dims && !inv_freq) ||
      norm_mode < 0 || norm_mode > 2 || (norm_mode && !qw) || !positions)
    return PTL_ERR_ARG;
  if (k_off >= 0 && (Hk <= 0 || Hv <= 0 || Dv <= 0 || page_size <= 0 || (norm_mode && !kw) ||
                     (slots && (!k_cache || !v_cache))))
    return PTL_ERR_ARG;
  const size_t floats = (size_t)Hq * Dk + (k_off >= 0 ? (size_t)Hk * Dk : 0) + Hq + (k_off >= 0 ? Hk : 0) + 2;
  const size_t lds = floats * sizeof(float);
  if (lds > 60 * 1024) return PTL_ERR_ARG;
  // slices of whole heads: about 512 workgroups in all when the tokens are few, one a token when
  // they are many
  const int heads = Hq + (k_off >= 0 ? Hk + Hv : 0);
  int slices = (512 + T_ - 1) / T_;
  if (slices > heads) slices = heads;
  if (slices < 1) slices = 1;
  const int heads_per_slice = (heads + slices - 1) / slices;
  slices = (heads + heads_per_slice - 1) / heads_per_slice;
  dim3 grid(T_, slices);
#define GO(TO)                                                                                        \
  {                                                                                                   \
    qkv_prepare_kernel<TO><<<grid, 256, lds, st>>>((TO*)q_out, p, ldp, q_off, k_off, v_off, qb, kb,   \
                                                   vb, norm_mode, qw, kw, eps, rot_dims, inv_freq,    \
                                                   mag, positions, slots, (TO*)k_cache,               \
                                                   (TO*)v_cache, Hq, Hk, Hv, Dk, Dv, page_size,       \
                                                   heads_per_slice);                                  \
    return ptl_launch_status();                                                                       \
  }
  if (dtype == PTL_DTYPE_F32) GO(float)
  if (dtype == PTL_DTYPE_BF16) GO(bf16_t)
#undef GO
  return PTL_ERR_ARG;
}

#define ACT_NONE 0
#define ACT_SIGMOID 1
#define ACT_SILU 2

template <typename TO>
__global__ void __launch_bounds__(256)
head_norm_gate_kernel(TO* __restrict__ out, long ldo, const float* __restrict__ a, int maps, float lam,
                      const float* __restrict__ w, int w_stride, float mult, const float* __restrict__ gate,
                      long ldg, int g_off, int act, float eps, int T_, int H, int Dv) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * 4 + wave;
  if (item >= (long)T_ * H) return;
  const int t = (int)(item / H), h = (int)(item - (long)t * H);
  const float* a1 = a + ((size_t)t * H * maps + (size_t)h * maps) * Dv;
  const float* a2 = a1 + Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += 64) {
    const float o = maps == 2 ? a1[d] - lam * a2[d] : a1[d];
    ss = fmaf(o, o, ss);
  }
  ss = wave_sum(ss);
  const float r = mult / sqrtf(ss / (float)Dv + eps);
  const float* g = gate ? gate + (size_t)t * ldg + g_off + (size_t)h * Dv : nullptr;
  TO* dst = out + (size_t)t * ldo + (size_t)h * Dv;
  for (int d = lane; d < Dv; d += 64) {
    float o = (maps == 2 ? a1[d] - lam * a2[d] : a1[d]) * r;
    if (w) o *= w[(size_t)h * w_stride + d];
    if (g) {
      const float z = g[d];
      const float sg = 1.0f / (1.0f + expf(-z));
      o *= act == ACT_SILU ? z * sg : sg;
    }
    dst[d] = from_float<TO>(o);
  }
}

// a float32 [T, H * maps, Dv] dense; out [T, ldo] (H * Dv columns used); gate float32 [T, ldg] read
// at columns g_off .. g_off + H * Dv, or null; w float32 (w_stride 0: [Dv] for all heads, Dv: [H, Dv]),
// or null.
extern "C" int ptl_head_norm_gate(void* out, long ldo, const float* a, int maps, float lam, const float* w,
                                  int w_stride, float mult, const float* gate, long ldg, int g_off, int act,
                                  float eps, int T_, int H, int Dv, int dtype, hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (H <= 0 || Dv <= 0 || maps < 1 || maps > 2 || act < 0 || act > 2 || (gate && act == ACT_NONE))
    return PTL_ERR_ARG;
  const long items = (long)T_ * H;
  const long blocks = (items + 3) / 4;
  if (blocks > 0x7fffffff) return PTL_ERR_ARG;
#define GO(TO)                                                                                         \
  {                                                                                                    \
    head_norm_gate_kernel<TO><<<(int)blocks, 256, 0, st>>>((TO*)out, ldo, a, maps, lam, w, w_stride,   \
                                                           mult, gate, ldg, g_off, act, eps, T_, H, Dv); \
    return ptl_launch_status();                                                                        \
  }
  if (dtype == PTL_DTYPE_F32) GO(float)
  if (dtype == PTL_DTYPE_BF16) GO(bf16_t)
#undef GO
  return PTL_ERR_ARG;
}
