// Matrix memory with exponential input and forget gates, kept in range by a running maximum.
//
//   i = cap tanh((x_i + b_i) / cap),  f = logsigmoid(cap tanh((x_f + b_f) / cap)),  q times Dk^-1/2;  per head:
//   m' = max(f + m, i);   S <- exp(f + m - m') S + exp(i - m') k v^T;   n <- the same with k alone;
//   o = S^T q / (max(|n . q|, exp(-m')) + denom_eps)
//   out = o / sqrt(mean_d o^2 + eps) * w * sigmoid(gate) * scale                 (mean over the head's Dv)
//
// Once m is known for every token the recurrence is a scan with a decay a_t = exp(f + m - m') and a value
// scale s_t = exp(i - m') per (token, head): the scan shared with the retention and state-space mixers
// (la::decay_scan_f32, retention.hip), segments and join included.  The normaliser n rides along as one
// more value column whose value is 1, so its read-out n . q is column Dv of the scan's output.
// State per sequence: [slots][H][Dv + 1][Dk] fp32 (value-column major, n last) and m [slots][H]; all zero
// at position 0.
//
// mm_prep_kernel: fp32 rows [q Dk^-1/2 | k] and [v | 1] per head.   mm_gates_kernel: a wave per
// (sequence portion, head) finds m for 64 tokens at a time by a scan over the lanes and writes
// (a_t, s_t, exp(-m_t)).   mm_out_kernel: denominator,
// unit norm, weight, gate, scale; a wave per (token, head).
#include "common.h"

namespace la {

int decay_scan_f32(const float* v, int ldv, const float* qk, int T, int nseq, int H, int Gqk, int Dk, int Dv,
                   const int* pos, const int* cu_q, const int* sslots, float* state, const float* tok_dec,
                   const float* tok_vs, int ldtok, float* o, float* seg, int max_rows, hipStream_t st);

template <typename AT>
__global__ __launch_bounds__(256) void mm_prep_kernel(const AT* __restrict__ src, long ld, int H, int Dk, int Dv, float qscale,
                                                      float* __restrict__ qk, float* __restrict__ va, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int per = 2 * H * Dk + H * (Dv + 1);
  const long t = e / per;
  const int c = (int)(e - t * per);
  const AT* row = src + t * ld;
  if (c < 2 * H * Dk) {
    qk[t * 2 * H * Dk + c] = (float)row[c] * (c < H * Dk ? qscale : 1.f);
  } else {
    const int u = c - 2 * H * Dk, h = u / (Dv + 1), d = u - h * (Dv + 1);
    va[t * H * (Dv + 1) + u] = d < Dv ? (float)row[2 * H * Dk + h * Dv + d] : 1.f;
  }
}

LA_DEV float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// A wave per (sequence portion, head), 64 tokens at a time: a token is the map m -> max(m + f, i), maps
// compose as (F1, I1) then (F2, I2) = (F1 + F2, max(I1 + F2, I2)), so an inclusive scan over the lanes
// gives every token's m from the chunk's incoming m.
template <typename AT>
__global__ __launch_bounds__(64) void mm_gates_kernel(const AT* __restrict__ src, long ld, int gcol, int H, int nseq,
                                                      const float* __restrict__ gate_b, float cap,
                                                      const int* __restrict__ pos, const int* __restrict__ cu_q,
                                                      const int* __restrict__ sslots, float* __restrict__ mstate,
                                                      float* __restrict__ gts) {
  const int seq = blockIdx.x / H, h = blockIdx.x - seq * H, lane = threadIdx.x;
  const int a = cu_q[seq], b = cu_q[seq + 1];
  if (b <= a) return;
  const int slot = sslots[seq];
  float m0 = (slot >= 0 && pos[a] != 0) ? mstate[(long)slot * H + h] : 0.f;
  const float bi = gate_b[h], bf = gate_b[H + h];
  for (int t0 = a; t0 < b; t0 += 64) {
    const int t = t0 + lane;
    const bool live = t < b;
    float ig = -INFINITY, fg = 0.f;        // a lane past the end is the identity map
    if (live) {
      const AT* row = src + (long)t * ld + gcol;
      ig = cap * tanhf(((float)row[h] + bi) / cap);
      fg = log_sigmoid(cap * tanhf(((float)row[H + h] + bf) / cap));
    }
    float F = fg, I = ig;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float Fp = __shfl_up(F, off, 64), Ip = __shfl_up(I, off, 64);
      if (lane >= off) {
        I = fmaxf(Ip + F, I);
        F = Fp + F;
      }
    }
    const float m = fmaxf(m0 + F, I);
    float mp = __shfl_up(m, 1, 64);
    if (lane == 0) mp = m0;
    if (live) {
      float* g = gts + (long)t * 3 * H;
      g[h] = expf(fg + mp - m);
      g[H + h] = expf(ig - m);
      g[2 * H + h] = expf(-m);
    }
    m0 = __shfl(m, min(63, b - 1 - t0), 64);
  }
  if (slot >= 0 && lane == 0) mstate[(long)slot * H + h] = m0;
}

template <typename AT>
__global__ __launch_bounds__(256) void mm_out_kernel(const float* __restrict__ o, const AT* __restrict__ src, long ld,
                                                     int ogcol, int H, int Dv, long rows, const float* __restrict__ gts,
                                                     const float* __restrict__ w, float eps, float denom_eps, float scale,
                                                     AT* __restrict__ out, long ldo) {
  const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int lane = threadIdx.x & 63;
  const long t = r / H;
  const int h = (int)(r - t * H);
  const float* orow = o + r * (Dv + 1);
  const float den = fmaxf(fabsf(orow[Dv]), gts[t * 3 * H + 2 * H + h]) + denom_eps;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += 64) {
    const float y = orow[d] / den;
    ss = fmaf(y, y, ss);
  }
  ss = wave_sum(ss);
  const float inv = scale / sqrtf(ss / (float)Dv + eps);
  const AT* g = src + t * ld + ogcol + (long)h * Dv;
  for (int d = lane; d < Dv; d += 64) {
    const float gv = (float)g[d];
    out[t * ldo + (long)h * Dv + d] = (AT)(orow[d] / den * inv * w[h * Dv + d] / (1.f + expf(-gv)));
  }
}

template <typename AT>
static int mm_launch(const AT* src, long ld, int T, int nseq, int H, int Dk, int Dv, const float* gate_b, float cap,
                     const float* nw, float eps, float denom_eps, float scale, const int* pos, const int* cu_q,
                     const int* sslots, float* mem, float* mstate, float* qk, float* va, float* gts, float* o, AT* out,
                     long ldo, float* seg, int max_rows, hipStream_t st) {
  const long total = (long)T * (2 * H * Dk + H * (Dv + 1));
  hipLaunchKernelGGL(mm_prep_kernel<AT>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, src, ld, H, Dk, Dv,
                     1.f / sqrtf((float)Dk), qk, va, total);
  const int gcol = 2 * H * Dk + 2 * H * Dv;
  hipLaunchKernelGGL(mm_gates_kernel<AT>, dim3(nseq * H), dim3(64), 0, st, src, ld, gcol, H, nseq, gate_b, cap,
                     pos, cu_q, sslots, mstate, gts);
  const int rc = decay_scan_f32(va, H * (Dv + 1), qk, T, nseq, H, H, Dk, Dv + 1, pos, cu_q, sslots, mem, gts, gts + H, 3 * H,
                                o, seg, max_rows, st);
  if (rc) return rc;
  const long rows = (long)T * H;
  hipLaunchKernelGGL(mm_out_kernel<AT>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const float*)o, src, ld,
                     2 * H * Dk + H * Dv, H, Dv, rows, (const float*)gts, nw, eps, denom_eps, scale, out, ldo);
  return (int)hipGetLastError();
}

}  // namespace la

extern "C" int la_matrix_memory(int f32, const void* src, long ld, int T, int nseq, int H, int Dk, int Dv, const void* gate_b,
                                float cap, const void* norm_w, float eps, float denom_eps, float scale, const void* pos,
                                const void* cu_q, const void* sslots, void* mem, void* mstate, int nslots, void* qk, void* va,
                                void* gts, void* o, void* out, long ldo, void* seg, int max_rows, void* stream) {
  using namespace la;
  if (T <= 0 || nseq <= 0 || H <= 0 || Dk <= 0 || Dv <= 0 || nslots <= 0 || cap <= 0.f ||
      ld < 2L * H * Dk + 2L * H * Dv + 2 * H || ldo < (long)H * Dv)
    return -1;
  if (!src || !gate_b || !norm_w || !pos || !cu_q || !sslots || !mem || !mstate || !qk || !va || !gts || !o || !out) return -2;
  hipStream_t st = (hipStream_t)stream;
  const int mr = max_rows > 0 ? max_rows : T;
  if (f32)
    return mm_launch<float>((const float*)src, ld, T, nseq, H, Dk, Dv, (const float*)gate_b, cap, (const float*)norm_w, eps,
                            denom_eps, scale, (const int*)pos, (const int*)cu_q, (const int*)sslots, (float*)mem,
                            (float*)mstate, (float*)qk, (float*)va, (float*)gts, (float*)o, (float*)out, ldo, (float*)seg, mr,
                            st);
  return mm_launch<bf16>((const bf16*)src, ld, T, nseq, H, Dk, Dv, (const float*)gate_b, cap, (const float*)norm_w, eps,
                         denom_eps, scale, (const int*)pos, (const int*)cu_q, (const int*)sslots, (float*)mem, (float*)mstate,
                         (float*)qk, (float*)va, (float*)gts, (float*)o, (bf16*)out, ldo, (float*)seg, mr, st);
}
