// Retention: linear attention with a fixed decay per head, no softmax and no denominator.
//
//   q_t, k_t rotated on their first `rot` dims (pair (i, i + rot / 2), angle pos * freq[i], fp32),
//   k_t times Dk^-1/2;   S_t = decay_h S_(t-1) + k_t v_t^T   (Dk x Dv, fp32);   o_t = S_t^T q_t
//   out_t = o_t / sqrt(mean_d o_t[d]^2 + eps) * silu(gate_t)          (mean over the head's Dv)
//
// The state of a sequence lives in a slot pool [slots][H][Dv][Dk] (value-column major) between
// launches: a portion starting at position 0 starts from zeros whatever the slot holds, any other
// portion from the slot, and every portion leaves its end state there.
//
// retention_rot_kernel: rotated q and scaled rotated k of every row, once, as fp32 [T][2][H][Dk].
// retention_scan_kernel: workgroup = (sequence portion, head, slice of value columns).  A column's
// Dk state entries sit in the registers of P lanes (R each, rows interleaved over the lanes, so LDS
// and state accesses of a lane group are consecutive), C columns a thread; tokens are staged through
// LDS in chunks (q, k, v) and scanned in order, o_t[c] reduced over the P lanes by shuffles.  P grows
// (narrower column slices, more workgroups) until a launch has about four workgroups per compute unit: a scan
// is a chain of dependent steps, so it is the number of resident waves that hides its latencies.  A
// decode batch is the same launch with one-token portions: it then streams each state once, which is
// its memory bound.  retention_out_kernel: the per-head unit norm and the gate.
//
// The scan also serves recurrences of the same shape whose decay changes from token to token and
// whose q / k rows are shared by groups of heads (state-space mixers, mamba2.hip):
//   S_t = a_(t,h) S_(t-1) + k_(t,g) (s_(t,h) v_(t,h))^T,   o_t = S_t^T q_(t,g)
// with a (tok_dec) and s (tok_vs) fp32 per (token, head) and Gqk groups; la::decay_scan_f32 is that entry.
#include "common.h"

namespace la {

constexpr int RT_NT = 256;
constexpr int RT_TC = 16;     // tokens staged per chunk
constexpr int RT_SEG = 128;   // rows per segment of a segmented portion
constexpr int RT_JOIN_MAXSEG = 1024;   // segments of one portion the join holds decay products for
enum { RT_WHOLE = 0, RT_LOCAL = 1, RT_FINAL = 2 };

// qk[t][0][h][d] = rotated q, qk[t][1][h][d] = rotated k * kscale (fp32): a thread per (row, head, pair or plain dim)
template <typename AT>
__global__ __launch_bounds__(256) void retention_rot_kernel(const AT* __restrict__ src, int ld, int H, int Dk,
                                                            const int* __restrict__ pos, const float* __restrict__ freqs,
                                                            float mag, int rot, float kscale, float* __restrict__ qk,
                                                            long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int half = rot >> 1, per = Dk - half;        // units per head: rot / 2 pairs, then Dk - rot plain dims
  const long th = e / per;
  const int u = (int)(e - th * per);
  const long t = th / H;
  const int h = (int)(th - t * H);
  const AT* q = src + t * ld + (long)h * Dk;
  const AT* k = q + (long)H * Dk;
  float* qo = qk + (t * 2 * H + h) * Dk;
  float* ko = qo + (long)H * Dk;
  if (u < half) {
    const float ang = (float)pos[t] * freqs[u];
    const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
    const float qu = (float)q[u], qw = (float)q[u + half], ku = (float)k[u], kw = (float)k[u + half];
    qo[u] = qu * cs - qw * sn;
    qo[u + half] = qw * cs + qu * sn;
    ko[u] = (ku * cs - kw * sn) * kscale;
    ko[u + half] = (kw * cs + ku * sn) * kscale;
  } else {
    const int d = u + half;
    qo[d] = (float)q[d];
    ko[d] = (float)k[d] * kscale;
  }
}

template <typename AT, int R, int C, bool EMIT>
__global__ __launch_bounds__(RT_NT) void retention_scan_kernel(
    const AT* __restrict__ src, int ld, long vcol0, const float* __restrict__ qk, int H, int Gqk, int Dk, int Dv,
    const int* __restrict__ pos, const int* __restrict__ cu_q, const int* __restrict__ sslots, float* __restrict__ state,
    const float* __restrict__ decay, const float* __restrict__ tok_dec, const float* __restrict__ tok_vs, int ldtok,
    float* __restrict__ o, int P, int mode, int L, int maxseg, float* __restrict__ seg_state) {
  extern __shared__ float lds[];
  const int DkP = P * R;                 // padded key width (rows beyond Dk hold zeros)
  const int cpw = RT_NT / P * C;         // value columns of this workgroup
  float* qs = lds;                       // [TC][DkP]
  float* ks = qs + RT_TC * DkP;          // [TC][DkP]
  float* vs = ks + RT_TC * DkP;          // [TC][cpw]
  float* dsh = vs + RT_TC * cpw;         // [TC] decay of every staged token (per-token decays)
  const int h = blockIdx.y, c0 = blockIdx.z * cpw;
  const int tid = threadIdx.x, part = tid % P, cg = tid / P, cb = c0 + cg * C;   // this thread's first column
  // mode RT_WHOLE: a workgroup scans a whole portion, slot state in and out.  Segmented portions:
  // RT_LOCAL scans a segment of L rows from a zero state and leaves its end state in seg_state (no
  // outputs, EMIT false); after retention_join_kernel has turned those into every segment's START
  // state, RT_FINAL scans the segment again from it and writes the outputs.
  int seq = blockIdx.x, a, b;
  float* st = nullptr;                   // state of column cb: [C][Dk]
  bool zero = true;
  if (mode == RT_WHOLE) {
    a = cu_q[seq];
    b = cu_q[seq + 1];
    if (b <= a) return;
    const int slot = sslots[seq];
    if (slot >= 0) st = state + (((long)slot * H + h) * Dv + cb) * Dk;
    zero = pos[a] == 0;
  } else {
    seq = blockIdx.x / maxseg;
    const int sidx = blockIdx.x - seq * maxseg;
    a = cu_q[seq] + sidx * L;
    const int b0 = cu_q[seq + 1];
    if (a >= b0) return;
    b = min(b0, a + L);
    int seg = sidx;
    for (int s2 = 0; s2 < seq; ++s2) seg += (cu_q[s2 + 1] - cu_q[s2] + L - 1) / L;
    st = seg_state + (((long)seg * H + h) * Dv + cb) * Dk;
    zero = mode == RT_LOCAL;
  }
  const float dec_h = decay ? decay[h] : 1.f;
  const int g = h / (H / Gqk);           // q / k rows are shared by the heads of a group
  float S[C][R];
#pragma unroll
  for (int ci = 0; ci < C; ++ci)
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int r = j * P + part;
      S[ci][j] = (st && !zero && r < Dk && cb + ci < Dv) ? st[(long)ci * Dk + r] : 0.f;
    }
  const long vcol = vcol0 + (long)h * Dv;
  for (int t0 = a; t0 < b; t0 += RT_TC) {
    const int n = min(RT_TC, b - t0);
    __syncthreads();
    for (int e = tid; e < n * DkP; e += RT_NT) {
      const int tt = e / DkP, d = e - tt * DkP;
      float qv = 0.f, kv = 0.f;
      if (d < Dk) {
        const float* row = qk + ((long)(t0 + tt) * 2 * Gqk + g) * Dk + d;
        if (EMIT) qv = row[0];
        kv = row[(long)Gqk * Dk];
      }
      if (EMIT) qs[e] = qv;
      ks[e] = kv;
    }
    for (int e = tid; e < n * cpw; e += RT_NT) {
      const int tt = e / cpw, cc = e - tt * cpw;
      float v = (c0 + cc < Dv) ? (float)src[(long)(t0 + tt) * ld + vcol + c0 + cc] : 0.f;
      if (tok_vs) v *= tok_vs[(long)(t0 + tt) * ldtok + h];
      vs[e] = v;
    }
    if (tok_dec && tid < n) dsh[tid] = tok_dec[(long)(t0 + tid) * ldtok + h];
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float dec = tok_dec ? dsh[tt] : dec_h;
      float vv[C], acc[C];
#pragma unroll
      for (int ci = 0; ci < C; ++ci) {
        vv[ci] = vs[tt * cpw + cg * C + ci];
        acc[ci] = 0.f;
      }
      const float* kr = ks + tt * DkP + part;
      const float* qr = qs + tt * DkP + part;
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const float kj = kr[j * P];
        const float qj = EMIT ? qr[j * P] : 0.f;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) {
          S[ci][j] = fmaf(dec, S[ci][j], kj * vv[ci]);
          if (EMIT) acc[ci] = fmaf(S[ci][j], qj, acc[ci]);
        }
      }
      if (EMIT) {
#pragma unroll
        for (int ci = 0; ci < C; ++ci) {
          float v = acc[ci];
          for (int w = P >> 1; w > 0; w >>= 1) v += __shfl_xor(v, w, 64);
          if (part == 0 && cb + ci < Dv) o[(long)(t0 + tt) * H * Dv + (long)h * Dv + cb + ci] = v;
        }
      }
    }
  }
  if (st && mode != RT_FINAL) {
#pragma unroll
    for (int ci = 0; ci < C; ++ci)
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const int r = j * P + part;
        if (r < Dk && cb + ci < Dv) st[(long)ci * Dk + r] = S[ci][j];
      }
  }
}

// Segment end states (from zero) -> segment start states, in place, and the portion's end state into
// its slot:  S_start(0) = slot state (zero at position 0),  S_start(s + 1) = decay^len(s) S_start(s) + S_local(s).
// A thread per state element of a (sequence, head).
__global__ __launch_bounds__(256) void retention_join_kernel(const int* __restrict__ pos, const int* __restrict__ cu_q,
                                                             const int* __restrict__ sslots, float* __restrict__ state,
                                                             const float* __restrict__ decay,
                                                             const float* __restrict__ tok_dec, int ldtok, int H,
                                                             long per_head, int L, float* __restrict__ seg_state) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const long e = (long)blockIdx.z * 256 + threadIdx.x;
  const int a = cu_q[seq], n = cu_q[seq + 1] - a;
  if (n <= 0) return;
  int seg = 0;
  for (int s2 = 0; s2 < seq; ++s2) seg += (cu_q[s2 + 1] - cu_q[s2] + L - 1) / L;
  const int slot = sslots[seq];
  float* st = (slot >= 0 && e < per_head) ? state + ((long)slot * H + h) * per_head + e : nullptr;
  float S = (st && pos[a] != 0) ? *st : 0.f;
  const float dec = decay ? decay[h] : 1.f, decL = powf(dec, (float)L);
  // per-token decays: every segment's product once per workgroup (a wave per segment, two shuffles
  // deep per 64 tokens), not once per state element
  __shared__ float sd[RT_JOIN_MAXSEG];
  const int nsegs = (n + L - 1) / L;
  if (tok_dec) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int s = wave; s < nsegs; s += 4) {
      const int len = min(L, n - s * L);
      float pd = 1.f;
      for (int t = lane; t < len; t += 64) pd *= tok_dec[(long)(a + s * L + t) * ldtok + h];
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) pd *= __shfl_xor(pd, o, 64);
      if (lane == 0) sd[s] = pd;
    }
    __syncthreads();
  }
  if (e >= per_head) return;
  for (int s = 0; s < nsegs; ++s) {
    const int len = min(L, n - s * L);
    float* p = seg_state + ((long)(seg + s) * H + h) * per_head + e;
    const float local = *p;
    *p = S;
    const float dseg = tok_dec ? sd[s] : (len == L ? decL : powf(dec, (float)len));
    S = fmaf(dseg, S, local);
  }
  if (st) *st = S;
}

// out[t][h][:] = o / sqrt(mean(o^2) + eps) * silu(gate): a wave per (token, head)
template <typename AT>
__global__ __launch_bounds__(256) void retention_out_kernel(const float* __restrict__ o, const AT* __restrict__ src, int ld,
                                                            long gcol, int H, int Dv, long rows, float eps,
                                                            AT* __restrict__ out) {
  const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int lane = threadIdx.x & 63;
  const long t = r / H;
  const int h = (int)(r - t * H);
  const float* orow = o + r * Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += 64) ss = fmaf(orow[d], orow[d], ss);
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)Dv + eps);
  const AT* g = src + t * ld + gcol + (long)h * Dv;
  for (int d = lane; d < Dv; d += 64) {
    const float gv = (float)g[d];
    out[r * Dv + d] = (AT)(orow[d] * inv * (gv / (1.f + expf(-gv))));
  }
}

// The scan over prepared rows: v from src (row stride ld, head h at column vcol0 + h Dv), q | k rows
// fp32 [T][2][Gqk][Dk], a fixed decay per head or tok_dec / tok_vs per (token, head) (row stride ldtok).
template <typename AT>
static int scan_core(const AT* src, int ld, long vcol0, int T, int nseq, int H, int Gqk, int Dk, int Dv, const int* pos,
                     const int* cu_q, const int* sslots, float* state, const float* decay, const float* tok_dec,
                     const float* tok_vs, int ldtok, const float* qk, float* o, float* seg, int max_rows, hipStream_t st) {
  // long batches of portions are cut into segments of RT_SEG rows scanned in parallel (two scans and a
  // join instead of one chain of T dependent steps); seg: [T / RT_SEG + nseq][H][Dv][Dk] fp32
  // (max_rows: the longest portion of the batch, known to the host; the grid holds that many segments a sequence)
  const bool segmented = seg != nullptr && T >= 8 * RT_SEG && max_rows >= 4 * RT_SEG &&
                         (max_rows + RT_SEG - 1) / RT_SEG <= RT_JOIN_MAXSEG;
  const int maxseg = (max_rows + RT_SEG - 1) / RT_SEG;
  const long chains = segmented ? (long)T / RT_SEG : nseq;
  // P lanes per group of C value columns (power of two), R rows per lane: P * R >= Dk with R <= 32; a
  // thread keeps C x R state entries, so a k / q value read from LDS feeds C multiply-adds (LDS
  // bandwidth bounds the scan otherwise).  More lanes per group while the launch has fewer than about
  // four workgroups per compute unit.
  const int Cc = Dv >= 64 ? 4 : 1;
  int P = 8;
  while (P < 64 && (Dk + P - 1) / P > (Cc == 4 ? 16 : 32)) P <<= 1;
  if ((Dk + P - 1) / P > 32) return -5;
  while (P < 64 && (Dk + P - 1) / P > 2 && chains * H * ((Dv + RT_NT / P * Cc - 1) / (RT_NT / P * Cc)) < 1024) P <<= 1;
  const int need = (Dk + P - 1) / P;
  const int cpw = RT_NT / P * Cc;
  const int nz = (Dv + cpw - 1) / cpw;
#define LA_RT_LAUNCH(RR, CC, EM, MODE, GX)                                                                            \
  {                                                                                                                   \
    const size_t shm = (size_t)(2 * RT_TC * P * RR + RT_TC * cpw + RT_TC) * sizeof(float);                            \
    if (shm > 150 * 1024) return -6;                                                                                  \
    if (shm > 48 * 1024)                                                                                              \
      (void)hipFuncSetAttribute((const void*)retention_scan_kernel<AT, RR, CC, EM>,                                   \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);                                \
    hipLaunchKernelGGL((retention_scan_kernel<AT, RR, CC, EM>), dim3(GX, H, nz), dim3(RT_NT), shm, st, src, ld,       \
                       vcol0, (const float*)qk, H, Gqk, Dk, Dv, pos, cu_q, sslots, state, decay, tok_dec, tok_vs,     \
                       ldtok, o, P, MODE, RT_SEG, maxseg, seg);                                                       \
  }
#define LA_RT_R(CC, EM, MODE, GX)                                                                                     \
  {                                                                                                                   \
    if (need <= 1) LA_RT_LAUNCH(1, CC, EM, MODE, GX)                                                                  \
    else if (need <= 2) LA_RT_LAUNCH(2, CC, EM, MODE, GX)                                                             \
    else if (need <= 4) LA_RT_LAUNCH(4, CC, EM, MODE, GX)                                                             \
    else if (need <= 8) LA_RT_LAUNCH(8, CC, EM, MODE, GX)                                                             \
    else if (need <= 16) LA_RT_LAUNCH(16, CC, EM, MODE, GX)                                                           \
    else LA_RT_LAUNCH(32, CC, EM, MODE, GX)                                                                           \
  }
#define LA_RT_SCAN(EM, MODE, GX)                                                                                      \
  {                                                                                                                   \
    if (Cc == 4) LA_RT_R(4, EM, MODE, GX)                                                                             \
    else LA_RT_R(1, EM, MODE, GX)                                                                                     \
  }
  if (!segmented) {
    LA_RT_SCAN(true, RT_WHOLE, nseq)
    return (int)hipGetLastError();
  }
  LA_RT_SCAN(false, RT_LOCAL, nseq * maxseg)
  const long per_head = (long)Dv * Dk;
  hipLaunchKernelGGL(retention_join_kernel, dim3(nseq, H, (unsigned)((per_head + 255) / 256)), dim3(256), 0, st, pos, cu_q,
                     sslots, state, decay, tok_dec, ldtok, H, per_head, RT_SEG, seg);
  LA_RT_SCAN(true, RT_FINAL, nseq * maxseg)
#undef LA_RT_SCAN
#undef LA_RT_R
#undef LA_RT_LAUNCH
  return (int)hipGetLastError();
}

template <typename AT>
static int launch_scan(const AT* src, int ld, int T, int nseq, int H, int Dk, int Dv, const int* pos, const int* cu_q,
                       const int* sslots, float* state, const float* decay, const float* freqs, float mag, int rot,
                       float* qk, float* o, float* seg, int max_rows, hipStream_t st) {
  const float kscale = 1.f / sqrtf((float)Dk);
  const long total = (long)T * H * (Dk - (rot >> 1));
  hipLaunchKernelGGL(retention_rot_kernel<AT>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, src, ld, H, Dk, pos,
                     freqs, mag, rot, kscale, qk, total);
  return scan_core<AT>(src, ld, 2L * H * Dk, T, nseq, H, H, Dk, Dv, pos, cu_q, sslots, state, decay, nullptr, nullptr, 0,
                       qk, o, seg, max_rows, st);
}

// Scan with per-token decays and value scales over fp32 rows (see the head of this file); seg as in
// la_retention ([T / RT_SEG + nseq][H][Dv][Dk] fp32, or null: whole portions only).
int decay_scan_f32(const float* v, int ldv, const float* qk, int T, int nseq, int H, int Gqk, int Dk, int Dv,
                   const int* pos, const int* cu_q, const int* sslots, float* state, const float* tok_dec,
                   const float* tok_vs, int ldtok, float* o, float* seg, int max_rows, hipStream_t st) {
  if (T <= 0 || nseq <= 0 || H <= 0 || Gqk <= 0 || H % Gqk || Dk <= 0 || Dv <= 0 || !tok_dec || ldtok < H) return -1;
  return scan_core<float>(v, ldv, 0L, T, nseq, H, Gqk, Dk, Dv, pos, cu_q, sslots, state, nullptr, tok_dec, tok_vs, ldtok,
                          qk, o, seg, max_rows > 0 ? max_rows : T, st);
}

}  // namespace la

extern "C" int la_retention(int f32, const void* src, int T, int nseq, int H, int Dk, int Dv, const void* pos,
                            const void* cu_q, const void* sslots, void* state, int nslots, const void* decay,
                            const void* freqs, float mag, int rot, float eps, void* qk, void* o, void* out, void* seg, int max_rows, void* stream) {
  using namespace la;
  if (T <= 0 || nseq <= 0 || H <= 0 || Dk <= 0 || Dv <= 0 || (rot & 1) || rot > Dk || nslots <= 0) return -1;
  if (!src || !pos || !cu_q || !sslots || !state || !decay || !freqs || !qk || !o || !out) return -2;
  hipStream_t st = (hipStream_t)stream;
  const int ld = 2 * H * Dk + 2 * H * Dv;
  const long gcol = 2L * H * Dk + (long)H * Dv, rows = (long)T * H;
  int rc;
  if (f32) {
    rc = launch_scan<float>((const float*)src, ld, T, nseq, H, Dk, Dv, (const int*)pos, (const int*)cu_q,
                            (const int*)sslots, (float*)state, (const float*)decay, (const float*)freqs, mag, rot,
                            (float*)qk, (float*)o, (float*)seg, max_rows > 0 ? max_rows : T, st);
    if (rc) return rc;
    hipLaunchKernelGGL(retention_out_kernel<float>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const float*)o,
                       (const float*)src, ld, gcol, H, Dv, rows, eps, (float*)out);
  } else {
    rc = launch_scan<bf16>((const bf16*)src, ld, T, nseq, H, Dk, Dv, (const int*)pos, (const int*)cu_q,
                           (const int*)sslots, (float*)state, (const float*)decay, (const float*)freqs, mag, rot,
                           (float*)qk, (float*)o, (float*)seg, max_rows > 0 ? max_rows : T, st);
    if (rc) return rc;
    hipLaunchKernelGGL(retention_out_kernel<bf16>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, (const float*)o,
                       (const bf16*)src, ld, gcol, H, Dv, rows, eps, (bf16*)out);
  }
  return (int)hipGetLastError();
}
