// Mixers that carry a matrix of fixed size from token to token instead of a cache that grows.
// Per head a matrix S [D, Dv] (keys x values), float32, kept in the request's state slot:
//
//   gated delta rule:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   matrix memory:     m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;
//                      n <- e^(f + m - m') n + e^(i - m') k;
//                      o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)           (m starts at 0)
//
// Every column of S (one value entry) goes its own way given k, q and the gates, so the columns
// are spread over the chip: a workgroup takes 16 columns of one head of one sequence, a column is
// held by 16 lanes (one row of a wave for the data-parallel lane moves), each lane with R rows of it
// in registers (D <= 16 R; rows beyond D stay zero). A step is R multiply-adds for each product
// and a sum over the 16 lanes; the tokens of a sequence are walked in order, 16 at a time through
// LDS (the next 16 are on their way from global memory meanwhile), so the result does not depend
// on how the sequence was cut into steps. n and m of the
// matrix memory are kept once per column block (every block carries the same values), so that no
// workgroup reads what another one writes.
//
// State of a slot: [H][blocks of 16 columns][16 D + D + 4] floats: S^T of the block (column
// after column, D rows each), then n [D], then m (matrix memory only; the delta rule leaves both
// untouched). The delta rule's slot also holds, behind that, the last taps - 1 inputs of its short
// convolutions [taps - 1][C].
//
// ptl_conv_prepare: for every token and head the short causal convolution over time of q, k and v
//   (inputs before the step's first token come from the slot), SiLU, and for q and k the unit norm
//   x / sqrt(sum(x^2) + 1e-6) (q also times D^-1/2), all float32.
// ptl_conv_tail_update: afterwards, the slot's last taps - 1 inputs.
// ptl_delta_scan / ptl_memory_scan: the recurrences; gates from the float32 projection.
// ptl_memory_scan_segments / ptl_delta_scan_segments: the same for steps with long portions, whose
//   rows are cut into segments that are walked side by side (described where they stand, below).
#include "common.h"
#include <math.h>

#define CHUNK 16

__device__ __forceinline__ float row16_sum(float v) {
  // the sum over the 16 lanes of a row, in every lane: rotations by 8, 4, 2 and 1 inside the row
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));
  return v;
}

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

#define MODE_DELTA 0
#define MODE_MEMORY 1

struct ScanArgs {
  float* out;            // [T, H, Dv]
  const float* q; long ldq;      // q[t * ldq + g * D + d]
  const float* k; long ldk;
  const float* v; long ldv;      // v[t * ldv + h * Dv + c]
  const float* ga; const float* gb; long ldg;   // raw gates [t * ldg + h]: delta (a, b); memory (i, f)
  const float* c0; const float* c1;              // [H]: delta (A_log, dt_bias); memory (i bias, f bias)
  float cap, qscale;
  float* state; long slot_stride;
  const int32_t* q_start; const int32_t* state_slots;
  int H, heads_per_qk, D, Dv;
};

template <int R, int MODE>
__global__ void __launch_bounds__(256) scan_kernel(ScanArgs A) {
  constexpr int DP = 16 * R;
  __shared__ float ks[CHUNK][DP], qs[CHUNK][DP], vs[CHUNK][16], os[CHUNK][16], g0s[CHUNK], g1s[CHUNK];
  const int tid = threadIdx.x;
  const int b = blockIdx.x, h = blockIdx.y, seq = blockIdx.z;
  const int row0 = A.q_start[seq];
  const int qlen = A.q_start[seq + 1] - row0;
  if (qlen <= 0) return;
  const int D = A.D, Dv = A.Dv;
  const int slot = A.state_slots[seq];
  const int nb = (Dv + 15) >> 4;
  const int block_floats = 16 * D + D + 4;
  float* st = A.state + (size_t)slot * A.slot_stride + ((size_t)h * nb + b) * block_floats;
  const int cg = tid >> 4, l = tid & 15;           // column of the block, lane of the column
  const int col = b * 16 + cg;
  const int g = h / A.heads_per_qk;
  float S[R], n[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = l * R + r;
    S[r] = (d < D && col < Dv) ? st[(size_t)cg * D + d] : 0.f;
    n[r] = (MODE == MODE_MEMORY && d < D) ? st[16 * D + d] : 0.f;
  }
  float m = MODE == MODE_MEMORY ? st[16 * D + D] : 0.f;

  // The next 16 tokens are fetched from global memory into registers while the current 16 are
  // worked on from LDS: a thread fetches R entries of k and of q (CHUNK * DP / 256), one of v
  // and, the first CHUNK threads, a token's two raw gates.
  float fk[R], fq[R], fv, fa, fb;
  auto fetch = [&](int t0) {
    const int steps = min(CHUNK, qlen - t0);
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = tid + 256 * j;
      const int t = i / DP, d = i - t * DP;
      fk[j] = 0.f;
      fq[j] = 0.f;
      if (t < steps && d < D) {
        const size_t row = (size_t)(row0 + t0 + t);
        fk[j] = A.k[row * A.ldk + (size_t)g * D + d];
        fq[j] = A.q[row * A.ldq + (size_t)g * D + d] * A.qscale;
      }
    }
    const int cc = b * 16 + l;
    fv = (cg < steps && cc < Dv) ? A.v[(size_t)(row0 + t0 + cg) * A.ldv + (size_t)h * Dv + cc] : 0.f;
    fa = fb = 0.f;
    if (tid < steps) {
      const size_t row = (size_t)(row0 + t0 + tid);
      fa = A.ga[row * A.ldg + h];
      fb = A.gb[row * A.ldg + h];
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = tid + 256 * j;
      const int t = i / DP, d = i - t * DP;
      ks[t][d] = fk[j];
      qs[t][d] = fq[j];
    }
    vs[cg][l] = fv;
    if (tid < CHUNK) {
      if (MODE == MODE_DELTA) {
        g0s[tid] = expf(-expf(A.c0[h]) * softplus_f(fa + A.c1[h]));      // decay
        g1s[tid] = 1.0f / (1.0f + expf(-fb));                             // beta
      } else {
        g0s[tid] = A.cap * tanhf((fa + A.c0[h]) / A.cap);                 // log input gate
        g1s[tid] = logsigmoid_f(A.cap * tanhf((fb + A.c1[h]) / A.cap));   // log forget gate
      }
    }
  };

  fetch(0);
  put();
  __syncthreads();
  for (int t0 = 0; t0 < qlen; t0 += CHUNK) {
    const int steps = min(CHUNK, qlen - t0);
    if (t0 + CHUNK < qlen) fetch(t0 + CHUNK);
    // a step's k, q, v and gates are read from LDS one step ahead of their use, into one of two
    // sets of registers in turn
    auto read = [&](float (&kr)[R], float (&qr)[R], float& v, float& ga, float& gb, int t) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        kr[r] = ks[t][l * R + r];
        qr[r] = qs[t][l * R + r];
      }
      v = vs[t][cg];
      ga = g0s[t];
      gb = g1s[t];
    };
    auto step = [&](const float (&kr)[R], const float (&qr)[R], float v, float ga, float gb, int t) {
      float o;
      if (MODE == MODE_DELTA) {
        const float decay = ga, beta = gb;
        float sk = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] *= decay;
          sk = fmaf(S[r], kr[r], sk);
        }
        sk = row16_sum(sk);
        const float u = beta * (v - sk);
        float sq = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] = fmaf(kr[r], u, S[r]);
          sq = fmaf(S[r], qr[r], sq);
        }
        o = row16_sum(sq);
      } else {
        const float gi = ga, gf = gb;
        const float m_new = fmaxf(gf + m, gi);
        const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
        m = m_new;
        const float tv = take * v;
        float sq = 0.f, nq = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] = fmaf(kr[r], tv, keep * S[r]);
          n[r] = fmaf(kr[r], take, keep * n[r]);
          sq = fmaf(S[r], qr[r], sq);
          nq = fmaf(n[r], qr[r], nq);
        }
        sq = row16_sum(sq);
        nq = row16_sum(nq);
        o = sq / (fmaxf(fabsf(nq), expf(-m_new)) + 1e-6f);
      }
      if (l == 0) os[t][cg] = o;
    };
    float k0[R], q0[R], k1[R], q1[R], v0, v1, a0, a1, b0, b1;
    read(k0, q0, v0, a0, b0, 0);
    for (int t = 0; t < steps; t += 2) {
      read(k1, q1, v1, a1, b1, (t + 1) & (CHUNK - 1));
      step(k0, q0, v0, a0, b0, t);
      if (t + 1 < steps) {
        read(k0, q0, v0, a0, b0, (t + 2) & (CHUNK - 1));
        step(k1, q1, v1, a1, b1, t + 1);
      }
    }
    __syncthreads();              // everyone has read this chunk; its results are in os
    {
      const int cc = b * 16 + l;
      if (cg < steps && cc < Dv) A.out[((size_t)(row0 + t0 + cg) * A.H + h) * Dv + cc] = os[cg][l];
    }
    if (t0 + CHUNK < qlen) put();
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = l * R + r;
    if (d < D && col < Dv) st[(size_t)cg * D + d] = S[r];
    if (MODE == MODE_MEMORY && cg == 0 && d < D) st[16 * D + d] = n[r];
  }
  if (MODE == MODE_MEMORY && tid == 0) st[16 * D + D] = m;
}

template <int MODE>
static int launch_scan(const ScanArgs& A, int n_seqs, hipStream_t st) {
  const int nb = (A.Dv + 15) / 16;
  if (A.D <= 0 || A.D > 256 || A.Dv <= 0 || A.H <= 0 || A.H > 65535 || n_seqs > 65535 ||
      A.heads_per_qk <= 0 || A.H % A.heads_per_qk)
    return PTL_ERR_ARG;
  dim3 grid(nb, A.H, n_seqs);
  const int R = (A.D + 15) / 16;
#define GO(RR)                                            \
  if (R <= RR) {                                          \
    scan_kernel<RR, MODE><<<grid, 256, 0, st>>>(A);       \
    return ptl_launch_status();                           \
  }
  GO(1) GO(2) GO(3) GO(4) GO(6) GO(8) GO(12) GO(16)
#undef GO
  return PTL_ERR_ARG;
}

// q, k float32 [T, G, D] (unit vectors), v float32 [T, H, Dv]; raw gates a and b float32 with row
// stride ldg, one a head; A_log, dt_bias float32 [H]. state: the slots, slot_stride floats each.
extern "C" int ptl_delta_scan(float* out, const float* q, const float* k, const float* v, const float* ga,
                              const float* gb, long ldg, const float* A_log, const float* dt_bias,
                              float* state, long slot_stride, const int32_t* q_start,
                              const int32_t* state_slots, int n_seqs, int H, int G, int D, int Dv,
                              hipStream_t st) {
  if (n_seqs <= 0) return PTL_OK;
  if (G <= 0 || H % G) return PTL_ERR_ARG;
  ScanArgs A{out, q, (long)G * D, k, (long)G * D, v, (long)H * Dv, ga, gb, ldg, A_log, dt_bias, 0.f, 1.f,
             state, slot_stride, q_start, state_slots, H, H / G, D, Dv};
  return launch_scan<MODE_DELTA>(A, n_seqs, st);
}

// q, k, v: columns of the float32 projection p [T, ldp] (H heads of D, D and Dv); raw gates i and f
// at columns i_off and f_off, their biases float32 [H]; q is multiplied by qscale.
extern "C" int ptl_memory_scan(float* out, const float* p, long ldp, int q_off, int k_off, int v_off,
                               int i_off, int f_off, const float* i_bias, const float* f_bias, float cap,
                               float qscale, float* state, long slot_stride, const int32_t* q_start,
                               const int32_t* state_slots, int n_seqs, int H, int D, int Dv,
                               hipStream_t st) {
  if (n_seqs <= 0) return PTL_OK;
  if (cap <= 0.f) return PTL_ERR_ARG;
  ScanArgs A{out, p + q_off, ldp, p + k_off, ldp, p + v_off, ldp, p + i_off, p + f_off, ldp, i_bias, f_bias,
             cap, qscale, state, slot_stride, q_start, state_slots, H, 1, D, Dv};
  return launch_scan<MODE_MEMORY>(A, n_seqs, st);
}

// ---- the matrix memory of a long prompt portion, segment by segment ---------------------------------
// The memory's transition is a scalar (S <- keep S + take k v^T), so a long portion need not be
// walked as one chain. Its rows are cut into segments of ``seg_len`` tokens:
//   the gates kernel      the scalar part alone, token by token (one workgroup a head and sequence):
//                         m, and keep = e^(f + m - m'), take = e^(i - m'), e^(-m') of every token;
//                         the final m goes to the slot
//   local pass            every segment but the last, side by side, from a zero state: what the
//                         segment adds (S, n) and the product of its keeps
//   ptl_memory_combine    the state each segment starts from: start(p + 1) = keeps(p) start(p) + added(p)
//   final pass            every segment, side by side, from its start state, with the read-outs;
//                         the last one leaves the state in the slot
// The same arithmetic a token as the walk in one chain, summed in another order.
struct SegArgs {
  float* out;                        // [T, H, Dv]
  const float* q; const float* k; const float* v; long ldp;     // columns of the projection
  const float* gates;                // [T, H, 4]: keep, take, e^(-m'), unused
  float qscale;
  float* state; long slot_stride;
  float* work;                       // [n_seqs * P][H][blocks][16 D + D + 4]: a segment's start state
  const int32_t* q_start; const int32_t* state_slots;
  int H, D, Dv, P, seg_len;
};

template <int R, bool FINAL>
__global__ void __launch_bounds__(256) memory_segment_kernel(SegArgs A) {
  constexpr int DP = 16 * R;
  __shared__ float ks[CHUNK][DP], qs[CHUNK][DP], vs[CHUNK][16], os[CHUNK][16], gs[CHUNK][4];
  const int tid = threadIdx.x;
  const int b = blockIdx.x, h = blockIdx.y;
  const int seq = blockIdx.z / A.P, seg = blockIdx.z - seq * A.P;
  const int row0 = A.q_start[seq];
  const int qlen = A.q_start[seq + 1] - row0;
  const int nseg = (qlen + A.seg_len - 1) / A.seg_len;
  if (qlen <= 0 || seg >= nseg || (!FINAL && seg == nseg - 1)) return;
  const int t_begin = seg * A.seg_len, t_end = min(qlen, t_begin + A.seg_len);
  const int D = A.D, Dv = A.Dv, H = A.H;
  const int nb = (Dv + 15) >> 4;
  const int block_floats = 16 * D + D + 4;
  auto work_at = [&](int p) {
    return A.work + (((size_t)(seq * A.P + p) * H + h) * nb + b) * block_floats;
  };
  const int cg = tid >> 4, l = tid & 15;
  const int col = b * 16 + cg;
  float S[R], n[R];
  {
    const float* from = work_at(seg);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = l * R + r;
      S[r] = (FINAL && d < D && col < Dv) ? from[(size_t)cg * D + d] : 0.f;
      n[r] = (FINAL && d < D) ? from[16 * D + d] : 0.f;
    }
  }
  float kept = 1.f;                    // the product of the segment's keeps (local pass)

  float fk[R], fq[R], fv, fg;
  auto fetch = [&](int t0) {
    const int steps = min(CHUNK, t_end - t0);
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = tid + 256 * j;
      const int t = i / DP, d = i - t * DP;
      fk[j] = 0.f;
      fq[j] = 0.f;
      if (t < steps && d < D) {
        const size_t row = (size_t)(row0 + t0 + t);
        fk[j] = A.k[row * A.ldp + (size_t)h * D + d];
        if (FINAL) fq[j] = A.q[row * A.ldp + (size_t)h * D + d] * A.qscale;
      }
    }
    const int cc = b * 16 + l;
    fv = (cg < steps && cc < Dv) ? A.v[(size_t)(row0 + t0 + cg) * A.ldp + (size_t)h * Dv + cc] : 0.f;
    fg = 0.f;
    if (tid < 4 * steps) fg = A.gates[((size_t)(row0 + t0 + (tid >> 2)) * H + h) * 4 + (tid & 3)];
  };
  auto put = [&]() {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = tid + 256 * j;
      const int t = i / DP, d = i - t * DP;
      ks[t][d] = fk[j];
      if (FINAL) qs[t][d] = fq[j];
    }
    vs[cg][l] = fv;
    if (tid < 4 * CHUNK) gs[tid >> 2][tid & 3] = fg;
  };
  fetch(t_begin);
  put();
  __syncthreads();
  for (int t0 = t_begin; t0 < t_end; t0 += CHUNK) {
    const int steps = min(CHUNK, t_end - t0);
    if (t0 + CHUNK < t_end) fetch(t0 + CHUNK);
    for (int t = 0; t < steps; ++t) {
      float kr[R], qr[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        kr[r] = ks[t][l * R + r];
        if (FINAL) qr[r] = qs[t][l * R + r];
      }
      const float keep = gs[t][0], take = gs[t][1];
      const float tv = take * vs[t][cg];
      if (FINAL) {
        float sq = 0.f, nq = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] = fmaf(kr[r], tv, keep * S[r]);
          n[r] = fmaf(kr[r], take, keep * n[r]);
          sq = fmaf(S[r], qr[r], sq);
          nq = fmaf(n[r], qr[r], nq);
        }
        sq = row16_sum(sq);
        nq = row16_sum(nq);
        const float o = sq / (fmaxf(fabsf(nq), gs[t][2]) + 1e-6f);
        if (l == 0) os[t][cg] = o;
      } else {
        kept *= keep;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] = fmaf(kr[r], tv, keep * S[r]);
          n[r] = fmaf(kr[r], take, keep * n[r]);
        }
      }
    }
    __syncthreads();
    if (FINAL) {
      const int cc = b * 16 + l;
      if (cg < steps && cc < Dv) A.out[((size_t)(row0 + t0 + cg) * H + h) * Dv + cc] = os[cg][l];
    }
    if (t0 + CHUNK < t_end) put();
    __syncthreads();
  }
  // local pass: what the segment adds, to where the next segment's start state will stand; final
  // pass of the last segment: the state, to the slot
  float* to = nullptr;
  if (!FINAL) to = work_at(seg + 1);
  else if (seg == nseg - 1)
    to = A.state + (size_t)A.state_slots[seq] * A.slot_stride + ((size_t)h * nb + b) * block_floats;
  if (to) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = l * R + r;
      if (d < D && col < Dv) to[(size_t)cg * D + d] = S[r];
      if (cg == 0 && d < D) to[16 * D + d] = n[r];
    }
    if (!FINAL && tid == 0) to[16 * D + D] = kept;
  }
}

__global__ void __launch_bounds__(256) memory_combine_kernel(SegArgs A) {
  const int b = blockIdx.x, h = blockIdx.y, seq = blockIdx.z;
  const int row0 = A.q_start[seq];
  const int qlen = A.q_start[seq + 1] - row0;
  if (qlen <= 0) return;
  const int nseg = (qlen + A.seg_len - 1) / A.seg_len;
  const int nb = (A.Dv + 15) >> 4;
  const int block_floats = 16 * A.D + A.D + 4;
  const int live = 16 * A.D + A.D;                  // S^T of the block and n
  const float* st = A.state + (size_t)A.state_slots[seq] * A.slot_stride + ((size_t)h * nb + b) * block_floats;
  for (int i = threadIdx.x; i < live; i += 256) {
    float cur = st[i];
    for (int p = 0; p < nseg; ++p) {
      float* w = A.work + (((size_t)(seq * A.P + p) * A.H + h) * nb + b) * block_floats;
      if (p > 0) cur = fmaf(w[live], cur, w[i]);      // keeps(p - 1) start(p - 1) + added(p - 1)
      w[i] = cur;
    }
  }
}

// One workgroup a (head, sequence): the log gates of 256 tokens side by side, the running maximum
// token by token (one wave, the gates read from LDS ahead of their use), then the three
// exponentials side by side. The final m goes to every column block's copy.
__global__ void __launch_bounds__(256)
memory_gates_kernel(float* __restrict__ gates, const float* __restrict__ gi_raw, const float* __restrict__ gf_raw,
                    long ldg, const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                    float* __restrict__ state, long slot_stride, const int32_t* __restrict__ q_start,
                    const int32_t* __restrict__ state_slots, int H, int D, int Dv) {
  __shared__ float gi_s[256], gf_s[256], before_s[256], after_s[256];
  const int h = blockIdx.x, seq = blockIdx.y, tid = threadIdx.x;
  const int row0 = q_start[seq];
  const int qlen = q_start[seq + 1] - row0;
  if (qlen <= 0) return;
  const int nb = (Dv + 15) >> 4;
  const int block_floats = 16 * D + D + 4;
  float* st = state + (size_t)state_slots[seq] * slot_stride + (size_t)h * nb * block_floats;
  float m = st[16 * D + D];
  // the raw gates of the next 256 tokens are on their way while the current ones are worked on
  float next_i = 0.f, next_f = 0.f;
  if (tid < qlen) {
    next_i = gi_raw[(size_t)(row0 + tid) * ldg + h];
    next_f = gf_raw[(size_t)(row0 + tid) * ldg + h];
  }
  const float bi = i_bias[h], bf = f_bias[h];
  for (int t0 = 0; t0 < qlen; t0 += 256) {
    const int steps = min(256, qlen - t0);
    const float raw_i = next_i, raw_f = next_f;
    if (t0 + 256 + tid < qlen) {
      next_i = gi_raw[(size_t)(row0 + t0 + 256 + tid) * ldg + h];
      next_f = gf_raw[(size_t)(row0 + t0 + 256 + tid) * ldg + h];
    }
    float gi = 0.f, gf = 0.f;
    if (tid < steps) {
      gi = cap * tanhf((raw_i + bi) / cap);
      gf = logsigmoid_f(cap * tanhf((raw_f + bf) / cap));
    }
    gi_s[tid] = gi;
    gf_s[tid] = gf;
    __syncthreads();
    if (tid < 64) {                       // (every lane the same values)
#pragma unroll 8
      for (int j = 0; j < steps; ++j) {
        const float m_new = fmaxf(gf_s[j] + m, gi_s[j]);
        before_s[j] = m;
        after_s[j] = m_new;
        m = m_new;
      }
    }
    __syncthreads();
    m = after_s[steps - 1];
    if (tid < steps) {
      const float m_before = before_s[tid], m_mine = after_s[tid];
      float* g = gates + ((size_t)(row0 + t0 + tid) * H + h) * 4;
      g[0] = expf(gf + m_before - m_mine);
      g[1] = expf(gi - m_mine);
      g[2] = expf(-m_mine);
      g[3] = m_mine;
    }
    __syncthreads();
  }
  for (int b = tid; b < nb; b += 256) st[(size_t)b * block_floats + 16 * D + D] = m;
}

// As ptl_memory_scan, for steps with long portions. gates float32 [T, H, 4] and work float32
// [n_seqs * P, H * blocks * (16 D + D + 4)] are workspaces of the caller; P >= the segments of the
// longest sequence of the step.
extern "C" int ptl_memory_scan_segments(float* out, const float* p, long ldp, int q_off, int k_off, int v_off,
                                        int i_off, int f_off, const float* i_bias, const float* f_bias,
                                        float cap, float qscale, float* state, long slot_stride,
                                        float* gates, float* work, int P, int seg_len,
                                        const int32_t* q_start, const int32_t* state_slots, int n_seqs,
                                        int H, int D, int Dv, hipStream_t st) {
  if (n_seqs <= 0) return PTL_OK;
  if (cap <= 0.f || P < 1 || seg_len < CHUNK || seg_len % CHUNK || D <= 0 || D > 256 || Dv <= 0 || H <= 0 ||
      H > 65535 || (long)n_seqs * P > 65535 || !gates || !work)
    return PTL_ERR_ARG;
  const int nb = (Dv + 15) / 16;
  memory_gates_kernel<<<dim3(H, n_seqs), 256, 0, st>>>(gates, p + i_off, p + f_off, ldp, i_bias, f_bias, cap,
                                                       state, slot_stride, q_start, state_slots, H, D, Dv);
  SegArgs A{out, p + q_off, p + k_off, p + v_off, ldp, gates, qscale, state, slot_stride, work, q_start,
            state_slots, H, D, Dv, P, seg_len};
  const dim3 grid(nb, H, n_seqs * P);
  const int R = (D + 15) / 16;
#define GO(RR)                                                          \
  if (R <= RR) {                                                        \
    if (P > 1) memory_segment_kernel<RR, false><<<grid, 256, 0, st>>>(A); \
    memory_combine_kernel<<<dim3(nb, H, n_seqs), 256, 0, st>>>(A);      \
    memory_segment_kernel<RR, true><<<grid, 256, 0, st>>>(A);           \
    return ptl_launch_status();                                         \
  }
  GO(1) GO(2) GO(3) GO(4) GO(6) GO(8) GO(12) GO(16)
#undef GO
  return PTL_ERR_ARG;
}

// ---- the delta rule of a long prompt portion, segment by segment --------------------------------------
// A step of the delta rule is S <- M S + beta k v^T with M = g (I - beta k k^T), the same M for every
// column of S. Over a segment S_end = W S_start + L, where L is what the segment makes of a zero
// state and W = M_last ... M_first is what it makes of the identity with the values left out: both
// come from the same walk, W as D more columns. So, as for the matrix memory:
//   local pass     every segment but the last, side by side: L (blocks of value columns) and W
//                  (blocks of the D columns of the identity)
//   combine        start(p + 1) = W(p) start(p) + L(p), segment after segment
//   final pass     every segment from its start state, with the read-outs; the last leaves the
//                  state in the slot
// Work area of a (sequence, segment, head): [value blocks][16][D] (start state; L of the segment
// before until the combine has run) then [key blocks][16][D] (W of the segment before, column c of
// W as row c).
struct DeltaSegArgs {
  float* out;                        // [T, H, Dv]
  const float* q; const float* k;    // [T, G, D] unit vectors
  const float* v;                    // [T, H, Dv]
  const float* ga; const float* gb; long ldg;     // raw gates a (decay), b (beta): [t * ldg + h]
  const float* A_log; const float* dt_bias;
  float* state; long slot_stride;
  float* work;
  const int32_t* q_start; const int32_t* state_slots;
  int H, heads_per_qk, D, Dv, P, seg_len;
};

template <int R, bool FINAL>
__global__ void __launch_bounds__(256) delta_segment_kernel(DeltaSegArgs A) {
  constexpr int DP = 16 * R;
  __shared__ float ks[CHUNK][DP], qs[CHUNK][DP], vs[CHUNK][16], os[CHUNK][16], g0s[CHUNK], g1s[CHUNK];
  const int tid = threadIdx.x;
  const int h = blockIdx.y;
  const int seq = blockIdx.z / A.P, seg = blockIdx.z - seq * A.P;
  const int row0 = A.q_start[seq];
  const int qlen = A.q_start[seq + 1] - row0;
  const int nseg = (qlen + A.seg_len - 1) / A.seg_len;
  if (qlen <= 0 || seg >= nseg || (!FINAL && seg == nseg - 1)) return;
  const int t_begin = seg * A.seg_len, t_end = min(qlen, t_begin + A.seg_len);
  const int D = A.D, Dv = A.Dv, H = A.H, G = H / A.heads_per_qk;
  const int nb = (Dv + 15) >> 4, nbk = (D + 15) >> 4;
  const bool is_w = !FINAL && (int)blockIdx.x >= nb;          // a block of W's columns
  const int b = is_w ? blockIdx.x - nb : blockIdx.x;
  const int ncols = is_w ? D : Dv;
  const size_t area = (size_t)(nb + nbk) * 16 * D;
  auto work_at = [&](int p) {
    return A.work + ((size_t)(seq * A.P + p) * H + h) * area + (is_w ? (size_t)nb * 16 * D : 0) +
           (size_t)b * 16 * D;
  };
  const int cg = tid >> 4, l = tid & 15;
  const int col = b * 16 + cg;
  const int g = h / A.heads_per_qk;
  float S[R];
  {
    const float* from = work_at(seg);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = l * R + r;
      if (FINAL) S[r] = (d < D && col < Dv) ? from[(size_t)cg * D + d] : 0.f;
      else S[r] = (is_w && d == col && d < D) ? 1.f : 0.f;
    }
  }
  float fk[R], fq[R], fv, fa, fb;
  auto fetch = [&](int t0) {
    const int steps = min(CHUNK, t_end - t0);
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = tid + 256 * j;
      const int t = i / DP, d = i - t * DP;
      fk[j] = 0.f;
      fq[j] = 0.f;
      if (t < steps && d < D) {
        const size_t at = ((size_t)(row0 + t0 + t) * G + g) * D + d;
        fk[j] = A.k[at];
        if (FINAL) fq[j] = A.q[at];
      }
    }
    const int cc = b * 16 + l;
    fv = (!is_w && cg < steps && cc < Dv) ? A.v[((size_t)(row0 + t0 + cg) * H + h) * Dv + cc] : 0.f;
    fa = fb = 0.f;
    if (tid < steps) {
      const size_t row = (size_t)(row0 + t0 + tid);
      fa = A.ga[row * A.ldg + h];
      fb = A.gb[row * A.ldg + h];
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = tid + 256 * j;
      const int t = i / DP, d = i - t * DP;
      ks[t][d] = fk[j];
      if (FINAL) qs[t][d] = fq[j];
    }
    vs[cg][l] = fv;
    if (tid < CHUNK) {
      g0s[tid] = expf(-expf(A.A_log[h]) * softplus_f(fa + A.dt_bias[h]));      // decay
      g1s[tid] = 1.0f / (1.0f + expf(-fb));                                     // beta
    }
  };
  fetch(t_begin);
  put();
  __syncthreads();
  for (int t0 = t_begin; t0 < t_end; t0 += CHUNK) {
    const int steps = min(CHUNK, t_end - t0);
    if (t0 + CHUNK < t_end) fetch(t0 + CHUNK);
    for (int t = 0; t < steps; ++t) {
      float kr[R], qr[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        kr[r] = ks[t][l * R + r];
        if (FINAL) qr[r] = qs[t][l * R + r];
      }
      const float decay = g0s[t], beta = g1s[t];
      float sk = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        S[r] *= decay;
        sk = fmaf(S[r], kr[r], sk);
      }
      sk = row16_sum(sk);
      const float u = beta * (vs[t][cg] - sk);
      if (FINAL) {
        float sq = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] = fmaf(kr[r], u, S[r]);
          sq = fmaf(S[r], qr[r], sq);
        }
        sq = row16_sum(sq);
        if (l == 0) os[t][cg] = sq;
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) S[r] = fmaf(kr[r], u, S[r]);
      }
    }
    __syncthreads();
    if (FINAL) {
      const int cc = b * 16 + l;
      if (cg < steps && cc < Dv) A.out[((size_t)(row0 + t0 + cg) * H + h) * Dv + cc] = os[cg][l];
    }
    if (t0 + CHUNK < t_end) put();
    __syncthreads();
  }
  float* to = nullptr;
  if (!FINAL) to = work_at(seg + 1);
  else if (seg == nseg - 1)
    to = A.state + (size_t)A.state_slots[seq] * A.slot_stride + ((size_t)h * nb + b) * (16 * D + D + 4);
  if (to) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = l * R + r;
      if (d < D && col < ncols) to[(size_t)cg * D + d] = S[r];
    }
  }
}

// start(0) = the slot's state; start(p) = W(p - 1) start(p - 1) + L(p - 1). A workgroup takes a block
// of 16 value columns of a head and walks the segments; a thread has one row d and CPG of the
// columns, so an entry of W (column e of W lies as row e: W[d][e] at e D + d) is loaded once, side by
// side with its neighbours in d, for all of them; the block's state lies in LDS as [e][16].
template <int CPG>
__global__ void __launch_bounds__(256) delta_combine_kernel(DeltaSegArgs A) {
  extern __shared__ float cur[];                  // [D][16]
  constexpr int GROUPS = 16 / CPG, DD = 256 / GROUPS;
  const int b = blockIdx.x, h = blockIdx.y, seq = blockIdx.z;
  const int row0 = A.q_start[seq];
  const int qlen = A.q_start[seq + 1] - row0;
  if (qlen <= 0) return;
  const int nseg = (qlen + A.seg_len - 1) / A.seg_len;
  const int D = A.D, H = A.H;
  const int nb = (A.Dv + 15) >> 4, nbk = (D + 15) >> 4;
  const size_t area = (size_t)(nb + nbk) * 16 * D;
  const float* st = A.state + (size_t)A.state_slots[seq] * A.slot_stride + ((size_t)h * nb + b) * (16 * D + D + 4);
  const int cols = min(16, A.Dv - b * 16);
  const int d = threadIdx.x % DD, c0 = (threadIdx.x / DD) * CPG;
  for (int i = threadIdx.x; i < 16 * D; i += 256) {
    const int c = i / D, e = i - c * D;
    cur[e * 16 + c] = c < cols ? st[i] : 0.f;
  }
  __syncthreads();
  for (int p = 0; p < nseg; ++p) {
    float* base = A.work + ((size_t)(seq * A.P + p) * H + h) * area;
    float* mine = base + (size_t)b * 16 * D;
    const float* W = base + (size_t)nb * 16 * D;
    float acc[CPG];
    if (d < D) {
      if (p == 0) {
#pragma unroll
        for (int j = 0; j < CPG; ++j) acc[j] = cur[d * 16 + c0 + j];
      } else {
#pragma unroll
        for (int j = 0; j < CPG; ++j) acc[j] = c0 + j < cols ? mine[(size_t)(c0 + j) * D + d] : 0.f;   // L
        // 32 entries of W on their way at a time: what binds here is how long one takes to come
        for (int e0 = 0; e0 < D; e0 += 32) {
          float w[32];
#pragma unroll
          for (int i = 0; i < 32; ++i) w[i] = e0 + i < D ? W[(size_t)(e0 + i) * D + d] : 0.f;
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            const int e = min(e0 + i, D - 1);
#pragma unroll
            for (int j = 0; j < CPG; ++j) acc[j] = fmaf(w[i], cur[e * 16 + c0 + j], acc[j]);
          }
        }
      }
    }
    __syncthreads();
    if (d < D) {
#pragma unroll
      for (int j = 0; j < CPG; ++j) {
        cur[d * 16 + c0 + j] = acc[j];
        if (c0 + j < cols) mine[(size_t)(c0 + j) * D + d] = acc[j];
      }
    }
    __syncthreads();
  }
}

// As ptl_delta_scan, for steps with long portions. work: float32 [n_seqs * P][H][(value blocks +
// key blocks) * 16 * D], a workspace of the caller; P >= the segments of the step's longest sequence.
extern "C" int ptl_delta_scan_segments(float* out, const float* q, const float* k, const float* v,
                                       const float* ga, const float* gb, long ldg, const float* A_log,
                                       const float* dt_bias, float* state, long slot_stride, float* work,
                                       int P, int seg_len, const int32_t* q_start,
                                       const int32_t* state_slots, int n_seqs, int H, int G, int D, int Dv,
                                       hipStream_t st) {
  if (n_seqs <= 0) return PTL_OK;
  if (G <= 0 || H % G || P < 1 || seg_len < CHUNK || seg_len % CHUNK || D <= 0 || D > 256 || Dv <= 0 ||
      H <= 0 || H > 65535 || (long)n_seqs * P > 65535 || !work)
    return PTL_ERR_ARG;
  const int nb = (Dv + 15) / 16, nbk = (D + 15) / 16;
  DeltaSegArgs A{out, q, k, v, ga, gb, ldg, A_log, dt_bias, state, slot_stride, work, q_start, state_slots,
                 H, H / G, D, Dv, P, seg_len};
  const int R = (D + 15) / 16;
  const size_t lds = (size_t)16 * D * sizeof(float);
#define GO(RR)                                                                                           \
  if (R <= RR) {                                                                                         \
    if (P > 1) delta_segment_kernel<RR, false><<<dim3(nb + nbk, H, n_seqs * P), 256, 0, st>>>(A);        \
    if (D <= 64) delta_combine_kernel<4><<<dim3(nb, H, n_seqs), 256, lds, st>>>(A);                      \
    else if (D <= 128) delta_combine_kernel<8><<<dim3(nb, H, n_seqs), 256, lds, st>>>(A);                \
    else delta_combine_kernel<16><<<dim3(nb, H, n_seqs), 256, lds, st>>>(A);                             \
    delta_segment_kernel<RR, true><<<dim3(nb, H, n_seqs * P), 256, 0, st>>>(A);                          \
    return ptl_launch_status();                                                                          \
  }
  GO(1) GO(2) GO(3) GO(4) GO(6) GO(8) GO(12) GO(16)
#undef GO
  return PTL_ERR_ARG;
}

// ---- the short convolutions in front of the delta rule -------------------------------------------
__device__ __forceinline__ int seq_of_row(const int32_t* __restrict__ q_start, int n_seqs, int t) {
  // the last sequence whose first row is not beyond t (sequences without rows share their start
  // with the one behind them); n_seqs for a row behind all sequences
  int lo = 0, hi = n_seqs;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__global__ void __launch_bounds__(256)
conv_prepare_kernel(float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ vv,
                    const float* __restrict__ p, long ldp, int x_off, const float* __restrict__ cw, int taps,
                    const float* __restrict__ state, long slot_stride, long tail_off,
                    const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots, int n_seqs,
                    int G, int H, int D, int Dv, float qscale) {
  extern __shared__ float buf[];
  __shared__ float scratch[16];
  const int t = blockIdx.x, blk = blockIdx.y, tid = threadIdx.x;
  const int C = 2 * G * D + H * Dv;
  const int seq = seq_of_row(q_start, n_seqs, t);
  int c0, n;
  float* dst;
  if (blk < G) { c0 = blk * D; n = D; dst = qn + ((size_t)t * G + blk) * D; }
  else if (blk < 2 * G) { c0 = G * D + (blk - G) * D; n = D; dst = kn + ((size_t)t * G + (blk - G)) * D; }
  else { c0 = 2 * G * D + (blk - 2 * G) * Dv; n = Dv; dst = vv + ((size_t)t * H + (blk - 2 * G)) * Dv; }
  if (seq >= n_seqs) {                      // a row that belongs to no sequence (padding)
    for (int d = tid; d < n; d += 256) dst[d] = 0.f;
    return;
  }
  const int row0 = q_start[seq];
  const int r = t - row0;
  const float* tail = state + (size_t)state_slots[seq] * slot_stride + tail_off;
  float ss = 0.f;
  for (int d = tid; d < n; d += 256) {
    const int c = c0 + d;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int i = r - (taps - 1) + j;
      const float x = i >= 0 ? p[(size_t)(row0 + i) * ldp + x_off + c] : tail[(size_t)(taps - 1 + i) * C + c];
      acc = fmaf(cw[(size_t)c * taps + j], x, acc);
    }
    const float y = acc / (1.0f + expf(-acc));
    buf[d] = y;
    ss = fmaf(y, y, ss);
  }
  if (blk >= 2 * G) {
    for (int d = tid; d < n; d += 256) dst[d] = buf[d];      // (each thread reads what it wrote)
    return;
  }
  ss = block_sum(ss, scratch);
  const float sc = (blk < G ? qscale : 1.f) / sqrtf(ss + 1e-6f);
  for (int d = tid; d < n; d += 256) dst[d] = buf[d] * sc;
}

// p float32 [T, ldp] with the inputs of the convolutions at columns x_off .. x_off + C, C = 2 G D +
// H Dv in the order q | k | v; cw float32 [C, taps]; the slot's tail [taps - 1, C] at tail_off.
extern "C" int ptl_conv_prepare(float* qn, float* kn, float* vv, const float* p, long ldp, int x_off,
                                const float* cw, int taps, const float* state, long slot_stride,
                                long tail_off, const int32_t* q_start, const int32_t* state_slots,
                                int n_seqs, int T_, int G, int H, int D, int Dv, float qscale,
                                hipStream_t st) {
  if (T_ <= 0) return PTL_OK;
  if (G <= 0 || H <= 0 || D <= 0 || Dv <= 0 || taps <= 0 || n_seqs <= 0 || 2 * G + H > 65535)
    return PTL_ERR_ARG;
  const size_t lds = (size_t)(D > Dv ? D : Dv) * sizeof(float);
  if (lds > 48 * 1024) return PTL_ERR_ARG;
  dim3 grid(T_, 2 * G + H);
  conv_prepare_kernel<<<grid, 256, lds, st>>>(qn, kn, vv, p, ldp, x_off, cw, taps, state, slot_stride,
                                               tail_off, q_start, state_slots, n_seqs, G, H, D, Dv, qscale);
  return ptl_launch_status();
}

__global__ void __launch_bounds__(256)
conv_tail_kernel(float* __restrict__ state, long slot_stride, long tail_off, const float* __restrict__ p,
                 long ldp, int x_off, const int32_t* __restrict__ q_start,
                 const int32_t* __restrict__ state_slots, int C, int taps) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int row0 = q_start[seq];
  const int qlen = q_start[seq + 1] - row0;
  if (qlen <= 0 || c >= C) return;
  float* tail = state + (size_t)state_slots[seq] * slot_stride + tail_off;
  // in order of rising i: an entry read from the old tail lies above the one being written
  for (int i = 0; i < taps - 1; ++i) {
    const int r = qlen - (taps - 1) + i;
    tail[(size_t)i * C + c] = r >= 0 ? p[(size_t)(row0 + r) * ldp + x_off + c] : tail[(size_t)(i + qlen) * C + c];
  }
}

extern "C" int ptl_conv_tail_update(float* state, long slot_stride, long tail_off, const float* p, long ldp,
                                    int x_off, const int32_t* q_start, const int32_t* state_slots,
                                    int n_seqs, int C, int taps, hipStream_t st) {
  if (n_seqs <= 0 || taps <= 1) return PTL_OK;
  if (C <= 0 || n_seqs > 65535) return PTL_ERR_ARG;
  dim3 grid((C + 255) / 256, n_seqs);
  conv_tail_kernel<<<grid, 256, 0, st>>>(state, slot_stride, tail_off, p, ldp, x_off, q_start, state_slots,
                                          C, taps);
  return ptl_launch_status();
}
