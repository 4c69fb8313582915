// Gated delta rule with one decay per head and key channel.
//
//   [q | k | v] rows pass a depthwise causal convolution over time and silu;  q, k (G heads of width Dk,
//   head h reads group h / (H / G)) become unit vectors, x / sqrt(sum x^2 + unit_eps), q times Dk^-1/2;
//   beta_h = sigmoid(.);  g_(h,d) = exp(-exp(a_log_h) softplus(dec_(h,d) + dt_bias_(h,d)));  per head, S (Dk x Dv):
//       S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
//   out = o / sqrt(mean_d o^2 + eps) * w_d * sigmoid(gate)                      (mean over the head's Dv)
//
// Per-sequence state between launches: the last taps - 1 rows of [q | k | v] before the convolution
// ([slots][taps - 1][C], the activation type) and S ([slots][H][Dv][Dk], fp32, value-column major).  A
// portion that starts at position 0 reads neither; every portion leaves both at its end.
//
// delta_prep_kernel: a workgroup per token.  Convolution + silu of every channel into LDS (inputs from
//   the portion's rows, then from the tail, zeros before position 0); a wave per q / k group forms both
//   unit vectors and k . q; fp32 rows out: [q | k] per group, v, the decays, (beta | k . q).  Batches of one
//   row per sequence advance the tail in the same launch (a thread owns its channels), other batches in
//   delta_tail_kernel afterwards, since rows of a portion read the old tail.  delta_prep8_kernel: the same
//   for bf16 rows of widths % 8, 8 channels a thread with 16-byte accesses and tap-major weights.
// delta_scan_kernel: workgroup = (sequence portion, head, slice of value columns).  The columns of S are
//   independent chains: column c needs a_c = (g S_c) . k and b_c = (g S_c) . q, then u_c = beta (v_c - a_c),
//   S_c <- g S_c + k u_c, and o_c = b_c + u_c (k . q), which is S_c . q after the write.  A column's Dk
//   entries sit in the registers of P lanes (R each, rows interleaved over the lanes), C columns a thread;
//   tokens are staged through LDS in chunks; a_c and b_c are reduced over the P lanes by shuffles.  A
//   decode batch is the same launch with one-token portions.
// delta_out_kernel: the per-head unit norm, its weight and the gate; a wave per (token, head).
#include "common.h"

namespace la {

constexpr int DR_NT = 256;
constexpr int DR_TC = 16;        // tokens staged per chunk
constexpr int DR_MAXTAPS = 16;

LA_DEV float dr_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

LA_DEV int portion_of(const int* __restrict__ cu_q, int nseq, int t) {
  int lo = 0, hi = nseq - 1;       // cu_q[seq] <= t < cu_q[seq + 1]
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}


// The value of lane (l xor W).  Within a row of 16 lanes the exchange is a data-parallel move on the
// vector unit (quad permutes and mirrors composed: i -> 7 - i -> i xor 4, i -> 15 - i -> i xor 8), which
// keeps the scan's reductions off the LDS crossbar; wider exchanges go through it.
template <int CTRL>
LA_DEV float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int W>
LA_DEV float lane_xor(float v) {
  if constexpr (W == 1) return dpp_move<0xB1>(v);                        // quad_perm [1, 0, 3, 2]
  else if constexpr (W == 2) return dpp_move<0x4E>(v);                   // quad_perm [2, 3, 0, 1]
  else if constexpr (W == 4) return dpp_move<0x1B>(dpp_move<0x141>(v));  // row_half_mirror, then quad_perm [3, 2, 1, 0]
  else if constexpr (W == 8) return dpp_move<0x141>(dpp_move<0x140>(v)); // row_mirror, then row_half_mirror
  else return __shfl_xor(v, W, 64);
}
template <int W, int N>
LA_DEV void butterfly_level(float (&a)[N], float (&b)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    a[i] += lane_xor<W>(a[i]);
    b[i] += lane_xor<W>(b[i]);
  }
}

template <typename AT>
__global__ __launch_bounds__(DR_NT) void delta_prep_kernel(
    const AT* __restrict__ src, long ld, const AT* __restrict__ dec, int H, int G, int Dk, int Dv, int taps,
    const float* __restrict__ w, const float* __restrict__ dt_bias, const float* __restrict__ a_log, float unit_eps,
    const int* __restrict__ pos, const int* __restrict__ cu_q, int nseq, const int* __restrict__ sslots,
    AT* __restrict__ tail, int single, float* __restrict__ qk, float* __restrict__ vf, float* __restrict__ gd,
    float* __restrict__ bq) {
  extern __shared__ float cv[];        // [C] convolved, activated channels of this token
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int Cqk = G * Dk, Cv = H * Dv, C = 2 * Cqk + Cv;
  const int seq = single ? t : portion_of(cu_q, nseq, t);
  const int a = cu_q[seq], p = pos[t], p0 = pos[a];
  const int slot = sslots[seq];
  const AT* st = (slot >= 0 && taps > 1) ? tail + (long)slot * (taps - 1) * C : nullptr;
  for (int c = tid; c < C; c += DR_NT) {
    float acc = 0.f;
    float cur[DR_MAXTAPS];             // this channel's inputs at positions p - taps + 1 .. p
#pragma unroll
    for (int j = 0; j < DR_MAXTAPS; ++j) {
      if (j < taps) {
        const int pj = p - (taps - 1) + j;
        float v = 0.f;
        if (pj >= p0) v = (float)src[(long)(a + pj - p0) * ld + c];
        else if (pj >= 0 && st) v = (float)st[(long)(pj - p0 + taps - 1) * C + c];
        cur[j] = v;
        acc = fmaf(w[(long)c * taps + j], v, acc);
      }
    }
    const float y = acc / (1.f + expf(-acc));
    cv[c] = y;
    if (c >= 2 * Cqk) vf[(long)t * Cv + (c - 2 * Cqk)] = y;
    if (single && slot >= 0 && taps > 1) {      // one row per sequence: the tail moves on by one position
      AT* sw = tail + (long)slot * (taps - 1) * C;
#pragma unroll
      for (int j = 1; j < DR_MAXTAPS; ++j)
        if (j < taps) sw[(long)(j - 1) * C + c] = (AT)cur[j];
    }
  }
  __syncthreads();
  const float qscale = 1.f / sqrtf((float)Dk);
  for (int g = wave; g < G; g += DR_NT / 64) {
    const float* q = cv + (long)g * Dk;
    const float* k = cv + Cqk + (long)g * Dk;
    float sq = 0.f, sk = 0.f, dot = 0.f;
    for (int d = lane; d < Dk; d += 64) {
      sq = fmaf(q[d], q[d], sq);
      sk = fmaf(k[d], k[d], sk);
      dot = fmaf(q[d], k[d], dot);
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    dot = wave_sum(dot);
    const float iq = qscale / sqrtf(sq + unit_eps), ik = 1.f / sqrtf(sk + unit_eps);
    float* qo = qk + ((long)t * 2 * G + g) * Dk;
    float* ko = qo + (long)G * Dk;
    for (int d = lane; d < Dk; d += 64) {
      qo[d] = q[d] * iq;
      ko[d] = k[d] * ik;
    }
    if (lane == 0) bq[(long)t * (H + G) + H + g] = dot * iq * ik;
  }
  for (int h = tid; h < H; h += DR_NT) {
    const float b = (float)src[(long)t * ld + C + h];
    bq[(long)t * (H + G) + h] = 1.f / (1.f + expf(-b));
  }
  for (int e = tid; e < H * Dk; e += DR_NT) {
    const int h = e / Dk;
    const float dt = dr_softplus((float)dec[(long)t * H * Dk + e] + dt_bias[e]);
    gd[(long)t * H * Dk + e] = expf(-expf(a_log[h]) * dt);
  }
}

// The same step for bf16 rows whose widths are multiples of 8 (key and value widths, the row stride): a
// thread takes 8 consecutive channels with 16-byte loads and reads the weights tap-major, w_t [taps][C],
// so a row's loads are in flight together instead of one round trip per channel.
__global__ __launch_bounds__(DR_NT) void delta_prep8_kernel(
    const bf16* __restrict__ src, long ld, const bf16* __restrict__ dec, int H, int G, int Dk, int Dv, int taps,
    const float* __restrict__ w_t, const float* __restrict__ dt_bias, const float* __restrict__ a_log, float unit_eps,
    const int* __restrict__ pos, const int* __restrict__ cu_q, int nseq, const int* __restrict__ sslots,
    bf16* __restrict__ tail, int single, float* __restrict__ qk, float* __restrict__ vf, float* __restrict__ gd,
    float* __restrict__ bq) {
  extern __shared__ float cv[];        // [C] convolved, activated channels of this token
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int Cqk = G * Dk, Cv = H * Dv, C = 2 * Cqk + Cv;
  const int seq = single ? t : portion_of(cu_q, nseq, t);
  const int a = cu_q[seq], p = pos[t], p0 = pos[a];
  const int slot = sslots[seq];
  const bf16* st = (slot >= 0 && taps > 1) ? tail + (long)slot * (taps - 1) * C : nullptr;
  for (int c = tid * 8; c < C; c += DR_NT * 8) {
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    bf16x8 cur[DR_MAXTAPS];
#pragma unroll
    for (int j = 0; j < DR_MAXTAPS; ++j) {
      if (j < taps) {
        const int pj = p - (taps - 1) + j;
        bf16x8 v;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (bf16)0.f;
        if (pj >= p0) v = *(const bf16x8*)(src + (long)(a + pj - p0) * ld + c);
        else if (pj >= 0 && st) v = *(const bf16x8*)(st + (long)(pj - p0 + taps - 1) * C + c);
        cur[j] = v;
        const float4 w0 = *(const float4*)(w_t + (long)j * C + c), w1 = *(const float4*)(w_t + (long)j * C + c + 4);
        acc[0] = fmaf(w0.x, (float)v[0], acc[0]);
        acc[1] = fmaf(w0.y, (float)v[1], acc[1]);
        acc[2] = fmaf(w0.z, (float)v[2], acc[2]);
        acc[3] = fmaf(w0.w, (float)v[3], acc[3]);
        acc[4] = fmaf(w1.x, (float)v[4], acc[4]);
        acc[5] = fmaf(w1.y, (float)v[5], acc[5]);
        acc[6] = fmaf(w1.z, (float)v[6], acc[6]);
        acc[7] = fmaf(w1.w, (float)v[7], acc[7]);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[i] = acc[i] / (1.f + expf(-acc[i]));
      cv[c + i] = acc[i];
    }
    if (c >= 2 * Cqk) {
      float4* o4 = (float4*)(vf + (long)t * Cv + (c - 2 * Cqk));
      o4[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
      o4[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
    if (single && slot >= 0 && taps > 1) {      // one row per sequence: the tail moves on by one position
      bf16* sw = tail + (long)slot * (taps - 1) * C;
#pragma unroll
      for (int j = 1; j < DR_MAXTAPS; ++j)
        if (j < taps) *(bf16x8*)(sw + (long)(j - 1) * C + c) = cur[j];
    }
  }
  __syncthreads();
  const float qscale = 1.f / sqrtf((float)Dk);
  for (int g = wave; g < G; g += DR_NT / 64) {
    const float* q = cv + (long)g * Dk;
    const float* k = cv + Cqk + (long)g * Dk;
    float sq = 0.f, sk = 0.f, dot = 0.f;
    for (int d = lane; d < Dk; d += 64) {
      sq = fmaf(q[d], q[d], sq);
      sk = fmaf(k[d], k[d], sk);
      dot = fmaf(q[d], k[d], dot);
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    dot = wave_sum(dot);
    const float iq = qscale / sqrtf(sq + unit_eps), ik = 1.f / sqrtf(sk + unit_eps);
    float* qo = qk + ((long)t * 2 * G + g) * Dk;
    float* ko = qo + (long)G * Dk;
    for (int d = lane; d < Dk; d += 64) {
      qo[d] = q[d] * iq;
      ko[d] = k[d] * ik;
    }
    if (lane == 0) bq[(long)t * (H + G) + H + g] = dot * iq * ik;
  }
  for (int h = tid; h < H; h += DR_NT) {
    const float b = (float)src[(long)t * ld + C + h];
    bq[(long)t * (H + G) + h] = 1.f / (1.f + expf(-b));
  }
  for (int e = tid * 8; e < H * Dk; e += DR_NT * 8) {
    const float ea = expf(a_log[e / Dk]);          // Dk % 8 == 0: the 8 channels share a head
    const bf16x8 dv = *(const bf16x8*)(dec + (long)t * H * Dk + e);
    const float4 b0 = *(const float4*)(dt_bias + e), b1 = *(const float4*)(dt_bias + e + 4);
    const float bb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = expf(-ea * dr_softplus((float)dv[i] + bb[i]));
    float4* o4 = (float4*)(gd + (long)t * H * Dk + e);
    o4[0] = make_float4(r[0], r[1], r[2], r[3]);
    o4[1] = make_float4(r[4], r[5], r[6], r[7]);
  }
}

// tail row i of a sequence <- the input at position end - (taps - 1) + i: a row of this portion, an
// older tail row, or zero before position 0.  A thread per (sequence, channel) reads all, then writes.
template <typename AT>
__global__ __launch_bounds__(DR_NT) void delta_tail_kernel(const AT* __restrict__ src, long ld, int C, int taps,
                                                           const int* __restrict__ pos, const int* __restrict__ cu_q,
                                                           const int* __restrict__ sslots, AT* __restrict__ tail) {
  const int seq = blockIdx.x, c = blockIdx.y * DR_NT + threadIdx.x;
  if (c >= C) return;
  const int a = cu_q[seq], n = cu_q[seq + 1] - a, slot = sslots[seq];
  if (n <= 0 || slot < 0) return;
  const int p0 = pos[a], pend = p0 + n;
  AT* st = tail + (long)slot * (taps - 1) * C;
  AT nv[DR_MAXTAPS];
#pragma unroll
  for (int i = 0; i < DR_MAXTAPS - 1; ++i) {
    if (i < taps - 1) {
      const int pi = pend - (taps - 1) + i;
      AT v = (AT)0.f;
      if (pi >= p0) v = src[(long)(a + pi - p0) * ld + c];
      else if (pi >= 0) v = st[(long)(pi - p0 + taps - 1) * C + c];
      nv[i] = v;
    }
  }
#pragma unroll
  for (int i = 0; i < DR_MAXTAPS - 1; ++i)
    if (i < taps - 1) st[(long)i * C + c] = nv[i];
}

template <int R, int C, int P>
__global__ __launch_bounds__(DR_NT) void delta_scan_kernel(
    const float* __restrict__ qk, const float* __restrict__ vf, const float* __restrict__ gd, const float* __restrict__ bq,
    int H, int G, int Dk, int Dv, const int* __restrict__ pos, const int* __restrict__ cu_q,
    const int* __restrict__ sslots, float* __restrict__ state, float* __restrict__ o) {
  extern __shared__ float lds[];
  constexpr int DkP = P * R;             // padded key width (rows beyond Dk hold zeros)
  constexpr int cpw = DR_NT / P * C;     // value columns of this workgroup
  float* qs = lds;                       // [TC][DkP]
  float* ks = qs + DR_TC * DkP;          // [TC][DkP]
  float* gs = ks + DR_TC * DkP;          // [TC][DkP]
  float* vs = gs + DR_TC * DkP;          // [TC][cpw]
  float* bs = vs + DR_TC * cpw;          // [TC][2]: beta, k . q
  const int seq = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * cpw;
  const int tid = threadIdx.x, part = tid % P, cg = tid / P, cb = c0 + cg * C;   // this thread's first column
  const int a = cu_q[seq], b = cu_q[seq + 1];
  if (b <= a) return;
  const int slot = sslots[seq];
  float* st = slot >= 0 ? state + (((long)slot * H + h) * Dv + cb) * Dk : nullptr;
  const bool zero = pos[a] == 0;
  const int g = h / (H / G);
  float S[C][R];
#pragma unroll
  for (int ci = 0; ci < C; ++ci)
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int r = j * P + part;
      S[ci][j] = (st && !zero && r < Dk && cb + ci < Dv) ? st[(long)ci * Dk + r] : 0.f;
    }
  for (int t0 = a; t0 < b; t0 += DR_TC) {
    const int n = min(DR_TC, b - t0);
    __syncthreads();
    for (int e = tid; e < n * DkP; e += DR_NT) {
      const int tt = e / DkP, d = e - tt * DkP;
      float qv = 0.f, kv = 0.f, gv = 1.f;
      if (d < Dk) {
        const float* row = qk + ((long)(t0 + tt) * 2 * G + g) * Dk + d;
        qv = row[0];
        kv = row[(long)G * Dk];
        gv = gd[((long)(t0 + tt) * H + h) * Dk + d];
      }
      qs[e] = qv;
      ks[e] = kv;
      gs[e] = gv;
    }
    for (int e = tid; e < n * cpw; e += DR_NT) {
      const int tt = e / cpw, cc = e - tt * cpw;
      vs[e] = (c0 + cc < Dv) ? vf[((long)(t0 + tt) * H + h) * Dv + c0 + cc] : 0.f;
    }
    if (tid < n) {
      bs[2 * tid] = bq[(long)(t0 + tid) * (H + G) + h];
      bs[2 * tid + 1] = bq[(long)(t0 + tid) * (H + G) + H + g];
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float beta = bs[2 * tt], kq = bs[2 * tt + 1];
      float ak[C], aq[C];
#pragma unroll
      for (int ci = 0; ci < C; ++ci) ak[ci] = aq[ci] = 0.f;
      const float* kr = ks + tt * DkP + part;
      const float* qr = qs + tt * DkP + part;
      const float* gr = gs + tt * DkP + part;
      float kj[R];
#pragma unroll
      for (int j = 0; j < R; ++j) {
        kj[j] = kr[j * P];
        const float qj = qr[j * P], gj = gr[j * P];
#pragma unroll
        for (int ci = 0; ci < C; ++ci) {
          const float s = gj * S[ci][j];
          S[ci][j] = s;
          ak[ci] = fmaf(s, kj[j], ak[ci]);
          aq[ci] = fmaf(s, qj, aq[ci]);
        }
      }
      // all 2 C sums move through every level of the butterfly together (the lane count is a template
      // parameter: the exchanges unroll and overlap instead of forming one chain of dependent shuffles)
      if constexpr (P >= 64) butterfly_level<32, C>(ak, aq);
      if constexpr (P >= 32) butterfly_level<16, C>(ak, aq);
      if constexpr (P >= 16) butterfly_level<8, C>(ak, aq);
      butterfly_level<4, C>(ak, aq);
      butterfly_level<2, C>(ak, aq);
      butterfly_level<1, C>(ak, aq);
#pragma unroll
      for (int ci = 0; ci < C; ++ci) {
        const float u = beta * (vs[tt * cpw + cg * C + ci] - ak[ci]);
#pragma unroll
        for (int j = 0; j < R; ++j) S[ci][j] = fmaf(kj[j], u, S[ci][j]);
        if (part == 0 && cb + ci < Dv) o[((long)(t0 + tt) * H + h) * Dv + cb + ci] = fmaf(u, kq, aq[ci]);
      }
    }
  }
  if (st) {
#pragma unroll
    for (int ci = 0; ci < C; ++ci)
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const int r = j * P + part;
        if (r < Dk && cb + ci < Dv) st[(long)ci * Dk + r] = S[ci][j];
      }
  }
}

// out[t][h][d] = o / sqrt(mean(o^2) + eps) * w[d] * sigmoid(gate): a wave per (token, head)
template <typename AT>
__global__ __launch_bounds__(256) void delta_out_kernel(const float* __restrict__ o, const AT* __restrict__ gate, int Dv,
                                                        long rows, int H, const float* __restrict__ w, float eps,
                                                        AT* __restrict__ out) {
  const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int lane = threadIdx.x & 63;
  const float* orow = o + r * Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += 64) ss = fmaf(orow[d], orow[d], ss);
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)Dv + eps);
  for (int d = lane; d < Dv; d += 64) {
    const float gv = (float)gate[r * Dv + d];
    out[r * Dv + d] = (AT)(orow[d] * inv * w[d] / (1.f + expf(-gv)));
  }
}

template <typename AT>
static int delta_launch(const AT* src, long ld, const AT* dec, const AT* gate, int T, int nseq, int H, int G, int Dk, int Dv,
                        int taps, const float* w, const float* w_t, const float* dt_bias, const float* a_log, const float* nw, float eps,
                        float unit_eps, const int* pos, const int* cu_q, const int* sslots, AT* tail, float* state,
                        int single, float* qk, float* vf, float* gd, float* bq, float* o, AT* out, hipStream_t st) {
  const int C = 2 * G * Dk + H * Dv;
  const size_t shm0 = (size_t)C * sizeof(float);
  if (shm0 > 150 * 1024) return -6;
  bool wide = false;
  if constexpr (sizeof(AT) == 2)
    wide = w_t && (Dk & 7) == 0 && (Dv & 7) == 0 && (ld & 7) == 0 && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dec & 15) == 0;
  if (wide) {
    if constexpr (sizeof(AT) == 2) {
      if (shm0 > 48 * 1024)
        (void)hipFuncSetAttribute((const void*)delta_prep8_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm0);
      hipLaunchKernelGGL(delta_prep8_kernel, dim3(T), dim3(DR_NT), shm0, st, (const bf16*)src, ld, (const bf16*)dec, H, G, Dk,
                         Dv, taps, w_t, dt_bias, a_log, unit_eps, pos, cu_q, nseq, sslots, (bf16*)tail, single, qk, vf, gd, bq);
    }
  } else {
    if (shm0 > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)delta_prep_kernel<AT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm0);
    hipLaunchKernelGGL(delta_prep_kernel<AT>, dim3(T), dim3(DR_NT), shm0, st, src, ld, dec, H, G, Dk, Dv, taps, w, dt_bias,
                       a_log, unit_eps, pos, cu_q, nseq, sslots, tail, single, qk, vf, gd, bq);
  }
  if (!single && taps > 1)
    hipLaunchKernelGGL(delta_tail_kernel<AT>, dim3(nseq, (C + DR_NT - 1) / DR_NT), dim3(DR_NT), 0, st, src, ld, C, taps, pos,
                       cu_q, sslots, tail);
  // P lanes per group of Cc value columns (power of two), R rows per lane: P * R >= Dk; a thread keeps
  // Cc x R state entries.  More lanes per group while the launch has fewer than about four workgroups
  // per compute unit (a scan is a chain of dependent steps, so resident waves hide its latencies), up to
  // 32: the sixth butterfly level costs more than the wider launch gains (4 x 2048 rows, 16 heads of
  // 128 x 128: 2.5 ms with 32 lanes, 3.3 ms with 64).
  // Cc: the most columns a thread (a k / q / g value read from LDS then feeds Cc chains) that still leaves
  // about two waves per SIMD at 16 lanes a group; a prompt batch of few sequences takes 1, a decode batch 4
  // (4 x 2048 rows, 16 heads of 128 x 128: 2.1 ms with 4 columns a thread, 1.6 with 2, 1.5 with 1).
  int Cc = 1;
  if (Dv >= 64)
    for (int c = 4; c >= 2; c >>= 1)
      if ((long)nseq * H * Dv / c * 16 / 64 >= 2048) {
        Cc = c;
        break;
      }
  int P = 8;
  while (P < 64 && (Dk + P - 1) / P > (Cc >= 2 ? 8 : 16)) P <<= 1;
  if ((Dk + P - 1) / P > 16) return -5;
  while (P < 32 && (Dk + P - 1) / P > 2 && (long)nseq * H * ((Dv + DR_NT / P * Cc - 1) / (DR_NT / P * Cc)) < 1024) P <<= 1;
  const int need = (Dk + P - 1) / P;
  const int cpw = DR_NT / P * Cc;
  const int nz = (Dv + cpw - 1) / cpw;
#define LA_DR_LAUNCH(RR, CC, PP)                                                                                     \
  {                                                                                                                  \
    const size_t shm = (size_t)(3 * DR_TC * PP * RR + DR_TC * cpw + 2 * DR_TC) * sizeof(float);                      \
    if (shm > 150 * 1024) return -6;                                                                                 \
    if (shm > 48 * 1024)                                                                                             \
      (void)hipFuncSetAttribute((const void*)delta_scan_kernel<RR, CC, PP>,                                          \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);                               \
    hipLaunchKernelGGL((delta_scan_kernel<RR, CC, PP>), dim3(nseq, H, nz), dim3(DR_NT), shm, st, (const float*)qk,   \
                       (const float*)vf, (const float*)gd, (const float*)bq, H, G, Dk, Dv, pos, cu_q, sslots, state, \
                       o);                                                                                           \
  }
#define LA_DR_P(RR, CC)                                                                                              \
  {                                                                                                                  \
    if (P == 8) LA_DR_LAUNCH(RR, CC, 8)                                                                              \
    else if (P == 16) LA_DR_LAUNCH(RR, CC, 16)                                                                       \
    else if (P == 32) LA_DR_LAUNCH(RR, CC, 32)                                                                       \
    else LA_DR_LAUNCH(RR, CC, 64)                                                                                    \
  }
#define LA_DR_R(CC)                                                                                                  \
  {                                                                                                                  \
    if (need <= 1) LA_DR_P(1, CC)                                                                                    \
    else if (need <= 2) LA_DR_P(2, CC)                                                                               \
    else if (need <= 4) LA_DR_P(4, CC)                                                                               \
    else if (need <= 8) LA_DR_P(8, CC)                                                                               \
    else LA_DR_P(16, CC)                                                                                             \
  }
  if (Cc == 4) LA_DR_R(4)
  else if (Cc == 2) LA_DR_R(2)
  else LA_DR_R(1)
#undef LA_DR_P
#undef LA_DR_R
#undef LA_DR_LAUNCH
  const long rows = (long)T * H;
  hipLaunchKernelGGL(delta_out_kernel<AT>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const float*)o, gate, Dv,
                     rows, H, nw, eps, out);
  return (int)hipGetLastError();
}

}  // namespace la

extern "C" int la_delta_rule(int f32, const void* src, long ld, const void* dec, const void* gate, int T, int nseq, int H,
                             int G, int Dk, int Dv, int taps, int nslots, const void* conv_w, const void* conv_wt,
                             const void* dt_bias,
                             const void* a_log, const void* norm_w, float eps, float unit_eps, const void* pos,
                             const void* cu_q, const void* sslots, void* tail, void* state, int single, void* qk, void* vf,
                             void* gd, void* bq, void* o, void* out, void* stream) {
  using namespace la;
  if (T <= 0 || nseq <= 0 || H <= 0 || G <= 0 || H % G || Dk <= 0 || Dv <= 0 || taps < 1 || taps > DR_MAXTAPS ||
      nslots <= 0 || ld < 2L * G * Dk + (long)H * Dv + H)
    return -1;
  if (!src || !dec || !gate || !conv_w || !dt_bias || !a_log || !norm_w || !pos || !cu_q || !sslots || !state || !qk ||
      !vf || !gd || !bq || !o || !out || (taps > 1 && !tail))
    return -2;
  if (single && T != nseq) return -3;
  hipStream_t st = (hipStream_t)stream;
  if (f32)
    return delta_launch<float>((const float*)src, ld, (const float*)dec, (const float*)gate, T, nseq, H, G, Dk, Dv, taps,
                               (const float*)conv_w, (const float*)conv_wt, (const float*)dt_bias, (const float*)a_log,
                               (const float*)norm_w, eps, unit_eps, (const int*)pos, (const int*)cu_q, (const int*)sslots, (float*)tail,
                               (float*)state, single, (float*)qk, (float*)vf, (float*)gd, (float*)bq, (float*)o,
                               (float*)out, st);
  return delta_launch<bf16>((const bf16*)src, ld, (const bf16*)dec, (const bf16*)gate, T, nseq, H, G, Dk, Dv, taps,
                            (const float*)conv_w, (const float*)conv_wt, (const float*)dt_bias, (const float*)a_log,
                            (const float*)norm_w, eps, unit_eps, (const int*)pos, (const int*)cu_q, (const int*)sslots, (bf16*)tail, (float*)state,
                            single, (float*)qk, (float*)vf, (float*)gd, (float*)bq, (float*)o, (bf16*)out, st);
}
