// State-space mixer with one decay per head (the state-space duality form), for batches of
// sequence portions with per-sequence state in slot pools.
//
//   projection row [z (H P) | x (H P) | B (G N) | C (G N) | dt (H)]
//   [x | B | C] <- silu(depthwise causal convolution over time + bias)   (taps, last = current token)
//   dt = softplus(dt + dt_bias);  a = exp(-exp(A_log) dt)                (fp32, per token and head)
//   S_t = a S_(t-1) + dt B_t x_t^T  (N x P, fp32);   y_t = S_t^T C_t + D x_t
//   out = unit-RMS over each of `norm_groups` equal parts of (y silu(z)), times a weight
//
// mamba2_conv_kernel: a workgroup per token; what precedes a portion comes from the sequence's
// convolution tail (the last taps - 1 rows of [x | B | C] before the convolution; zeros before
// position 0).  It writes fp32 x rows, fp32 [C | B] rows in the scan's q | k layout, and (dt, a).
// Batches of one row per sequence advance the tail in the same launch (a thread owns its channels);
// other batches in mamba2_tail_kernel afterwards, since rows of a portion read the old tail.
// The recurrence is la::decay_scan_f32 (retention.hip): q = C, k = B (shared by the heads of a group),
// v = dt x, decay a; state [slots][H][P][N] fp32, zero at position 0.
// mamba2_out_kernel: skip term, gate, grouped norm; a workgroup per (token, norm group).
#include "common.h"

namespace la {

int decay_scan_f32(const float* v, int ldv, const float* qk, int T, int nseq, int H, int Gqk, int Dk, int Dv,
                   const int* pos, const int* cu_q, const int* sslots, float* state, const float* tok_dec,
                   const float* tok_vs, int ldtok, float* o, float* seg, int max_rows, hipStream_t st);

constexpr int M2_NT = 256;
constexpr int M2_MAXTAPS = 16;

LA_DEV float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

template <typename AT>
__global__ __launch_bounds__(M2_NT) void mamba2_conv_kernel(
    const AT* __restrict__ src, int ld, int H, int inner, int GN, int taps, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const int* __restrict__ pos, const int* __restrict__ cu_q, int nseq, const int* __restrict__ sslots,
    AT* __restrict__ tail, int single, float* __restrict__ xs, float* __restrict__ cb, float* __restrict__ dtd) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const int C = inner + 2 * GN;
  int seq;
  if (single) {
    seq = t;
  } else {            // the portion that holds row t: cu_q[seq] <= t < cu_q[seq + 1]
    int lo = 0, hi = nseq - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
    }
    seq = lo;
  }
  const int a = cu_q[seq], p = pos[t], p0 = pos[a];
  const int slot = sslots[seq];
  const AT* st = (slot >= 0 && taps > 1) ? tail + (long)slot * (taps - 1) * C : nullptr;
  const AT* xbc = src + inner;         // [x | B | C] columns of a row
  for (int c = tid; c < C; c += M2_NT) {
    float acc = bias ? bias[c] : 0.f;
    float cur[M2_MAXTAPS];             // this channel's inputs at positions p - taps + 1 .. p
#pragma unroll
    for (int j = 0; j < M2_MAXTAPS; ++j) {
      if (j < taps) {
        const int pj = p - (taps - 1) + j;
        float v = 0.f;
        if (pj >= p0) v = (float)xbc[(long)(a + pj - p0) * ld + c];
        else if (pj >= 0 && st) v = (float)st[(long)(pj - p0 + taps - 1) * C + c];
        cur[j] = v;
        acc = fmaf(w[(long)c * taps + j], v, acc);
      }
    }
    const float y = silu(acc);
    if (c < inner) xs[(long)t * inner + c] = y;
    else if (c < inner + GN) cb[(long)t * 2 * GN + GN + (c - inner)] = y;   // B: the scan's k rows
    else cb[(long)t * 2 * GN + (c - inner - GN)] = y;                        // C: the scan's q rows
    if (single && slot >= 0 && taps > 1) {      // one row per sequence: the tail moves on by one position
      AT* sw = tail + (long)slot * (taps - 1) * C;
#pragma unroll
      for (int j = 1; j < M2_MAXTAPS; ++j)
        if (j < taps) sw[(long)(j - 1) * C + c] = (AT)cur[j];
    }
  }
  for (int h = tid; h < H; h += M2_NT) {
    const float dt = softplus_f((float)src[(long)t * ld + 2 * inner + 2 * GN + h] + dt_bias[h]);
    dtd[(long)t * 2 * H + h] = dt;
    dtd[(long)t * 2 * H + H + h] = expf(-expf(a_log[h]) * dt);
  }
}

// The same step for widths that are multiples of 8 (x, B and C regions each): a thread takes 8
// consecutive channels with 16-byte loads (bf16) and reads the weights tap-major, w_t [taps][C].
template <typename AT>
__global__ __launch_bounds__(M2_NT) void mamba2_conv8_kernel(
    const AT* __restrict__ src, int ld, int H, int inner, int GN, int taps, const float* __restrict__ w_t,
    const float* __restrict__ bias, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const int* __restrict__ pos, const int* __restrict__ cu_q, int nseq, const int* __restrict__ sslots,
    AT* __restrict__ tail, int single, float* __restrict__ xs, float* __restrict__ cb, float* __restrict__ dtd) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const int C = inner + 2 * GN;
  int seq;
  if (single) {
    seq = t;
  } else {
    int lo = 0, hi = nseq - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
    }
    seq = lo;
  }
  const int a = cu_q[seq], p = pos[t], p0 = pos[a];
  const int slot = sslots[seq];
  AT* st = (slot >= 0 && taps > 1) ? tail + (long)slot * (taps - 1) * C : nullptr;
  const AT* xbc = src + inner;
  auto load8 = [&](const AT* q, float* v) {
    if constexpr (sizeof(AT) == 2) {
      const bf16x8 r = *(const bf16x8*)q;
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = (float)r[k];
    } else {
      const float4 r0 = *(const float4*)q, r1 = *(const float4*)(q + 4);
      v[0] = r0.x; v[1] = r0.y; v[2] = r0.z; v[3] = r0.w; v[4] = r1.x; v[5] = r1.y; v[6] = r1.z; v[7] = r1.w;
    }
  };
  auto store8 = [&](AT* q, const float* v) {
    if constexpr (sizeof(AT) == 2) {
      bf16x8 r;
#pragma unroll
      for (int k = 0; k < 8; ++k) r[k] = (bf16)v[k];
      *(bf16x8*)q = r;
    } else {
      *(float4*)q = make_float4(v[0], v[1], v[2], v[3]);
      *(float4*)(q + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
  };
  for (int c = tid * 8; c < C; c += M2_NT * 8) {
    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = bias ? bias[c + k] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int pj = p - (taps - 1) + j;
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (pj >= p0) load8(xbc + (long)(a + pj - p0) * ld + c, v);
      else if (pj >= 0 && st) load8(st + (long)(pj - p0 + taps - 1) * C + c, v);
      const float4 w0 = *(const float4*)(w_t + (long)j * C + c), w1 = *(const float4*)(w_t + (long)j * C + c + 4);
      acc[0] = fmaf(w0.x, v[0], acc[0]); acc[1] = fmaf(w0.y, v[1], acc[1]);
      acc[2] = fmaf(w0.z, v[2], acc[2]); acc[3] = fmaf(w0.w, v[3], acc[3]);
      acc[4] = fmaf(w1.x, v[4], acc[4]); acc[5] = fmaf(w1.y, v[5], acc[5]);
      acc[6] = fmaf(w1.z, v[6], acc[6]); acc[7] = fmaf(w1.w, v[7], acc[7]);
      // one row per sequence: the tail moves on by one position (tail row j - 1 <- the input of tap j)
      if (single && st && j >= 1) store8(st + (long)(j - 1) * C + c, v);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = silu(acc[k]);
    float* dst;
    if (c < inner) dst = xs + (long)t * inner + c;
    else if (c < inner + GN) dst = cb + (long)t * 2 * GN + GN + (c - inner);
    else dst = cb + (long)t * 2 * GN + (c - inner - GN);
    *(float4*)dst = make_float4(acc[0], acc[1], acc[2], acc[3]);
    *(float4*)(dst + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
  }
  for (int h = tid; h < H; h += M2_NT) {
    const float dt = softplus_f((float)src[(long)t * ld + 2 * inner + 2 * GN + h] + dt_bias[h]);
    dtd[(long)t * 2 * H + h] = dt;
    dtd[(long)t * 2 * H + H + h] = expf(-expf(a_log[h]) * dt);
  }
}

// tail row i of a sequence <- the input at position end - (taps - 1) + i: a row of this portion, an
// older tail row, or zero before position 0.  A thread per (sequence, channel) reads all, then writes.
template <typename AT>
__global__ __launch_bounds__(M2_NT) void mamba2_tail_kernel(const AT* __restrict__ src, int ld, int inner, int C, int taps,
                                                            const int* __restrict__ pos, const int* __restrict__ cu_q,
                                                            const int* __restrict__ sslots, AT* __restrict__ tail) {
  const int seq = blockIdx.x, c = blockIdx.y * M2_NT + threadIdx.x;
  if (c >= C) return;
  const int a = cu_q[seq], n = cu_q[seq + 1] - a, slot = sslots[seq];
  if (n <= 0 || slot < 0) return;
  const int p0 = pos[a], pend = p0 + n;
  AT* st = tail + (long)slot * (taps - 1) * C;
  AT nv[M2_MAXTAPS];
#pragma unroll
  for (int i = 0; i < M2_MAXTAPS - 1; ++i) {
    if (i < taps - 1) {
      const int pi = pend - (taps - 1) + i;
      AT v = (AT)0.f;
      if (pi >= p0) v = src[(long)(a + pi - p0) * ld + inner + c];
      else if (pi >= 0) v = st[(long)(pi - p0 + taps - 1) * C + c];
      nv[i] = v;
    }
  }
#pragma unroll
  for (int i = 0; i < M2_MAXTAPS - 1; ++i)
    if (i < taps - 1) st[(long)i * C + c] = nv[i];
}

template <typename AT>
__global__ __launch_bounds__(M2_NT) void mamba2_out_kernel(const float* __restrict__ o, const float* __restrict__ xs,
                                                           const AT* __restrict__ src, int ld, int inner, int P, int gs,
                                                           const float* __restrict__ dskip, const float* __restrict__ nw,
                                                           float eps, AT* __restrict__ out) {
  __shared__ float red[M2_NT / 64];
  const int t = blockIdx.x, c0 = blockIdx.y * gs, tid = threadIdx.x;
  auto gated = [&](int c) {
    const float y = fmaf(dskip[c / P], xs[(long)t * inner + c], o[(long)t * inner + c]);
    const float z = (float)src[(long)t * ld + c];
    return y * (z / (1.f + expf(-z)));
  };
  // groups of up to 16 columns a thread keep their gated values in registers between the two passes
  constexpr int KEEP = 16;
  const bool keep = gs <= KEEP * M2_NT;
  float held[KEEP];
  float ss = 0.f;
  if (keep) {
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int c = c0 + tid + k * M2_NT;
      held[k] = c < c0 + gs ? gated(c) : 0.f;
      ss = fmaf(held[k], held[k], ss);
    }
  } else {
    for (int c = c0 + tid; c < c0 + gs; c += M2_NT) {
      const float y = gated(c);
      ss = fmaf(y, y, ss);
    }
  }
  ss = block_sum<M2_NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)gs + eps);
  if (keep) {
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      const int c = c0 + tid + k * M2_NT;
      if (c < c0 + gs) out[(long)t * inner + c] = (AT)(held[k] * inv * nw[c]);
    }
  } else {
    for (int c = c0 + tid; c < c0 + gs; c += M2_NT) out[(long)t * inner + c] = (AT)(gated(c) * inv * nw[c]);
  }
}

template <typename AT>
static int run(const AT* src, int T, int nseq, int H, int P, int N, int G, int taps, const float* conv_w,
               const float* conv_wt, const float* conv_b, const float* dt_bias, const float* a_log, const float* dskip, const float* nw,
               int norm_groups, float eps, const int* pos, const int* cu_q, const int* sslots, AT* tail, float* state,
               int single, float* xs, float* cb, float* dtd, float* o, AT* out, float* seg, int max_rows, hipStream_t st) {
  const int inner = H * P, GN = G * N, C = inner + 2 * GN, ld = 2 * inner + 2 * GN + H;
  if (conv_wt && !(inner & 7) && !(GN & 7) && !(ld & 7))
    hipLaunchKernelGGL(mamba2_conv8_kernel<AT>, dim3(T), dim3(M2_NT), 0, st, src, ld, H, inner, GN, taps, conv_wt, conv_b,
                       dt_bias, a_log, pos, cu_q, nseq, sslots, tail, single, xs, cb, dtd);
  else
    hipLaunchKernelGGL(mamba2_conv_kernel<AT>, dim3(T), dim3(M2_NT), 0, st, src, ld, H, inner, GN, taps, conv_w, conv_b,
                       dt_bias, a_log, pos, cu_q, nseq, sslots, tail, single, xs, cb, dtd);
  if (!single && taps > 1)
    hipLaunchKernelGGL(mamba2_tail_kernel<AT>, dim3(nseq, (C + M2_NT - 1) / M2_NT), dim3(M2_NT), 0, st, src, ld, inner, C,
                       taps, pos, cu_q, sslots, tail);
  const int rc = decay_scan_f32(xs, inner, cb, T, nseq, H, G, N, P, pos, cu_q, sslots, state, dtd + H, dtd, 2 * H, o, seg,
                                max_rows, st);
  if (rc) return rc;
  hipLaunchKernelGGL(mamba2_out_kernel<AT>, dim3(T, norm_groups), dim3(M2_NT), 0, st, (const float*)o, (const float*)xs, src,
                     ld, inner, P, inner / norm_groups, dskip, nw, eps, out);
  return (int)hipGetLastError();
}

}  // namespace la

// conv_wt: the convolution weights tap-major, [taps][C] (or null).  single: every sequence brings one row (cu_q = 0, 1, 2, ...).  xs [T, H P], cb [T, 2 G N], dtd [T, 2 H], o [T, H P]:
// fp32 scratch; seg: segment states of long batches as in la_retention, or null.
extern "C" int la_mamba2(int f32, const void* src, int T, int nseq, int H, int P, int N, int G, int taps, int nslots,
                         const void* conv_w, const void* conv_wt, const void* conv_b, const void* dt_bias, const void* a_log, const void* dskip,
                         const void* nw, int norm_groups, float eps, const void* pos, const void* cu_q, const void* sslots,
                         void* tail, void* state, int single, void* xs, void* cb, void* dtd, void* o, void* out, void* seg,
                         int max_rows, void* stream) {
  using namespace la;
  if (T <= 0 || nseq <= 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G || taps < 1 || taps > M2_MAXTAPS || nslots <= 0 ||
      norm_groups < 1 || (H * P) % norm_groups || (single && nseq != T))
    return -1;
  if (!src || !conv_w || !dt_bias || !a_log || !dskip || !nw || !pos || !cu_q || !sslots || !state || !xs || !cb || !dtd ||
      !o || !out || (taps > 1 && !tail))
    return -2;
  hipStream_t st = (hipStream_t)stream;
  if (f32)
    return run<float>((const float*)src, T, nseq, H, P, N, G, taps, (const float*)conv_w, (const float*)conv_wt, (const float*)conv_b,
                      (const float*)dt_bias, (const float*)a_log, (const float*)dskip, (const float*)nw, norm_groups, eps,
                      (const int*)pos, (const int*)cu_q, (const int*)sslots, (float*)tail, (float*)state, single, (float*)xs,
                      (float*)cb, (float*)dtd, (float*)o, (float*)out, (float*)seg, max_rows, st);
  return run<bf16>((const bf16*)src, T, nseq, H, P, N, G, taps, (const float*)conv_w, (const float*)conv_wt, (const float*)conv_b,
                   (const float*)dt_bias, (const float*)a_log, (const float*)dskip, (const float*)nw, norm_groups, eps,
                   (const int*)pos, (const int*)cu_q, (const int*)sslots, (bf16*)tail,
                   (float*)state, single, (float*)xs, (float*)cb, (float*)dtd, (float*)o, (bf16*)out, (float*)seg, max_rows, st);
}
