// Attention whose scores are reshaped before the softmax, over the paged K/V pools:
//
//   s_g(i, j)  = softcap * tanh(scale * q_g(i) . k(j) / softcap)          (softcap 0: none)
//                - slope_g * (i - j)                                       (slopes null: none)
//   s'_h(i, j) = sum_g talk[h][g] * s_g(i, j)                              (talk null: identity)
//   visible j:   j <= i, same chunk of `chunk` positions (chunk 0: all), within `window` (0: all)
//   o_h(i)     = gate_h(i) * sum_j softmax_j(s'_h(i, .)) v(j)              (gate null: 1)
//
// The head mix couples all heads of a (query, key) pair, so one workgroup owns ONE query row with
// every head: per tile of 64 keys it forms the H x 64 raw scores, mixes them through LDS, runs one
// online-softmax step per head (a wave per head, a lane per key) and accumulates P.V with threads
// spread over (head, value channel).  Query rows are independent (row -> sequence, position), so a
// launch takes prompt portions and single decoded tokens alike.  K and V rows of key and value
// width Dk / Dv may differ; the row kernel also takes pools without V pages, where the first Dv
// columns of a key row are its value.  Scores, softmax and the accumulators are fp32; q, K, V, gate logits
// and the output are the activation type (bf16 or fp32).
#include "common.h"

namespace la {

constexpr int AM_KT = 64;     // keys per tile = lanes of the softmax wave
constexpr int AM_NT = 256;
constexpr int AM_MAXO = 32;   // output accumulators per thread: H * Dv <= AM_NT * AM_MAXO

// q (fp32, LDS) . k (a cache row).  vec: the row is 16-byte aligned and D a multiple of the vector
template <typename AT>
LA_DEV float dot_row(const float* __restrict__ q, const AT* __restrict__ k, int D, bool vec);

template <>
LA_DEV float dot_row<float>(const float* __restrict__ q, const float* __restrict__ k, int D, bool vec) {
  float a = 0.f;
  int d = 0;
  if (vec)
    for (; d + 4 <= D; d += 4) {
      const float4 kv = *(const float4*)(k + d);
      a = fmaf(q[d], kv.x, a); a = fmaf(q[d + 1], kv.y, a); a = fmaf(q[d + 2], kv.z, a); a = fmaf(q[d + 3], kv.w, a);
    }
  for (; d < D; ++d) a = fmaf(q[d], k[d], a);
  return a;
}
template <>
LA_DEV float dot_row<bf16>(const float* __restrict__ q, const bf16* __restrict__ k, int D, bool vec) {
  float a = 0.f;
  int d = 0;
  if (vec)
    for (; d + 8 <= D; d += 8) {
      const bf16x8 kv = *(const bf16x8*)(k + d);
#pragma unroll
      for (int e = 0; e < 8; ++e) a = fmaf(q[d + e], (float)kv[e], a);
    }
  for (; d < D; ++d) a = fmaf(q[d], (float)k[d], a);
  return a;
}

template <typename AT>
__global__ __launch_bounds__(AM_NT) void attn_mix_rows_kernel(
    const AT* __restrict__ q, const AT* __restrict__ kc, const AT* __restrict__ vc, const int* __restrict__ row_seq,
    const int* __restrict__ pos, const int* __restrict__ bt, int maxb, int H, int G, int Dk, int Dv, int BS,
    float scale, float softcap, const float* __restrict__ slopes, const float* __restrict__ talk, int chunk,
    int window, const AT* __restrict__ gate, int ldg, AT* __restrict__ out, const float* __restrict__ dbias, int nbias,
    const float* __restrict__ sink) {
  extern __shared__ float lds[];
  float* qs = lds;                       // [H][Dk]
  float* s1 = qs + H * Dk;               // [H][KT] raw scores
  float* s2 = s1 + H * AM_KT;            // [H][KT] mixed scores, then probabilities
  float* mrun = s2 + H * AM_KT;          // [H] running max
  float* lrun = mrun + H;                // [H] running sum
  float* alpha = lrun + H;               // [H] rescale of this tile
  const int r = blockIdx.x, tid = threadIdx.x;
  const int i = pos[r];
  const int* tab = bt + (long)row_seq[r] * maxb;
  const int rep = H / G;
  const bool vec = (Dk * sizeof(AT)) % 16 == 0;
  for (int e = tid; e < H * Dk; e += AM_NT) qs[e] = (float)q[(long)r * H * Dk + e];
  // a sink is a logit without key or value: the running (max, sum) start at (sink, 1) instead of (-inf, 0)
  for (int h = tid; h < H; h += AM_NT) { mrun[h] = sink ? sink[h] : -INFINITY; lrun[h] = sink ? 1.f : 0.f; }
  int lo = 0;
  if (chunk > 0) lo = (i / chunk) * chunk;
  if (window > 0) lo = max(lo, i - window + 1);
  const int HV = H * Dv;
  float acc[AM_MAXO];
#pragma unroll
  for (int e = 0; e < AM_MAXO; ++e) acc[e] = 0.f;
  __syncthreads();
  for (int j0 = lo; j0 <= i; j0 += AM_KT) {
    const int nk = min(AM_KT, i + 1 - j0);
    // raw scores of every (head, key) pair of the tile
    for (int e = tid; e < H * AM_KT; e += AM_NT) {
      const int h = e / AM_KT, jj = e - h * AM_KT;
      float s = -INFINITY;
      if (jj < nk) {
        const int j = j0 + jj, blk = tab[j / BS], off = j % BS, g = h / rep;
        s = dot_row<AT>(qs + h * Dk, kc + (((long)blk * G + g) * BS + off) * Dk, Dk, vec) * scale;
        if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        if (slopes) s -= slopes[h] * (float)(i - j);
        if (dbias) s += dbias[(long)min(i - j, nbias - 1) * H + h];
      }
      s1[e] = s;
    }
    __syncthreads();
    if (talk) {
      for (int e = tid; e < H * AM_KT; e += AM_NT) {
        const int h = e / AM_KT, jj = e - h * AM_KT;
        float m = -INFINITY;
        if (jj < nk) {
          m = 0.f;
          for (int g = 0; g < H; ++g) m = fmaf(talk[h * H + g], s1[g * AM_KT + jj], m);
        }
        s2[e] = m;
      }
    } else {
      for (int e = tid; e < H * AM_KT; e += AM_NT) s2[e] = s1[e];
    }
    __syncthreads();
    // one online-softmax step per head: a wave per head, a lane per key
    for (int h = tid >> 6; h < H; h += AM_NT / 64) {
      const int lane = tid & 63;
      const float s = s2[h * AM_KT + lane];
      const float mo = mrun[h];
      const float mn = fmaxf(mo, wave_max(s));
      const float p = (s == -INFINITY) ? 0.f : __expf(s - mn);
      const float ps = wave_sum(p);
      s2[h * AM_KT + lane] = p;
      if (lane == 0) {
        const float a = (mo == -INFINITY) ? 0.f : __expf(mo - mn);
        alpha[h] = a;
        lrun[h] = lrun[h] * a + ps;
        mrun[h] = mn;
      }
    }
    __syncthreads();
    // o[h][d] = o[h][d] * alpha[h] + sum_jj p[h][jj] * V[j][g(h)][d]
#pragma unroll
    for (int e = 0; e < AM_MAXO; ++e) {
      const int o = tid + e * AM_NT;
      if (o < HV) {
        const int h = o / Dv, d = o - h * Dv, g = h / rep;
        float a = acc[e] * alpha[h];
        if (vc) {
          for (int jj = 0; jj < nk; ++jj) {
            const int j = j0 + jj, blk = tab[j / BS], off = j % BS;
            a = fmaf(s2[h * AM_KT + jj], (float)vc[((((long)blk * G + g) * (BS >> 3) + (off >> 3)) * Dv + d) * 8 + (off & 7)], a);
          }
        } else {   // no V pages: a key row's first Dv columns are its value (latent caches)
          for (int jj = 0; jj < nk; ++jj) {
            const int j = j0 + jj, blk = tab[j / BS], off = j % BS;
            a = fmaf(s2[h * AM_KT + jj], (float)kc[(((long)blk * G + g) * BS + off) * Dk + d], a);
          }
        }
        acc[e] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int e = 0; e < AM_MAXO; ++e) {
    const int o = tid + e * AM_NT;
    if (o < HV) {
      const int h = o / Dv;
      float v = acc[e] / lrun[h];
      if (gate) v *= 1.f / (1.f + __expf(-(float)gate[(long)r * ldg + h]));
      out[(long)r * HV + o] = (AT)v;
    }
  }
}


// ------------------------------------------------------------------------------------------------
// Prompt portions in bf16 on the matrix cores.  Workgroup = 16 consecutive query rows of one
// sequence portion x ALL heads, NW waves; per tile of 32 keys:
//   A  S_h = Q_h K_g^T per head (a wave owns HPW consecutive heads, so heads of one kv group
//      share their K fragments), MFMA 16x16x32 bf16 with both operands read straight from global
//      memory in operand layout (16 B per lane), Q fragments kept in registers over the key loop;
//      scale, softcap and the distance slope applied to the fp32 accumulators -> LDS s1[h][q][key]
//   B  head mix s'_h = sum_g talk[h][g] s_g as an fp32 MFMA 16x16x4 (A = talk, B = 16 (q, key)
//      columns of s1) -- scores never leave fp32 -- written back in place with the visibility mask
//      (a wave owns its column blocks, and reads all of a block before it writes)
//   C  one online-softmax step per (head, query) row: a thread per row over the 32 keys;
//      probabilities -> LDS as bf16 in A-operand layout
//   D  O_h += P_h V_g, MFMA 16x16x32 bf16, V read from the pages transposed per 8 keys
// Epilogue: 1 / l, the sigmoid head gate, bf16 store.  HPW = heads per wave, NDV = Dv / 16.
constexpr int AT_KT = 32;
constexpr int AT_SS = AT_KT + 1;   // fp32 score row stride: rows spread over the LDS banks
constexpr int AT_PS = AT_KT + 8;   // bf16 probability row stride: 16-byte aligned rows

template <int NW, int HPW, int NDV>
__global__ __launch_bounds__(NW * 64) void attn_mix_tile_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
    const int* __restrict__ tiles, const int* __restrict__ cu_q, const int* __restrict__ pos,
    const int* __restrict__ bt, int maxb, int H, int G, int Dk, int Dv, int BS, float scale, float softcap,
    const float* __restrict__ slopes, const float* __restrict__ talk, int chunk, int window,
    const bf16* __restrict__ gate, int ldg, bf16* __restrict__ out, int nsplit, float* __restrict__ part_o,
    float* __restrict__ part_ml, const float* __restrict__ dbias, int nbias, const float* __restrict__ sink) {
  extern __shared__ float lds[];
  float* s1 = lds;                           // [H][16][AT_SS]
  float* mrun = s1 + H * 16 * AT_SS;         // [H * 16]
  float* lrun = mrun + H * 16;
  float* alpha = lrun + H * 16;
  bf16* pb = (bf16*)(alpha + H * 16);        // [H][16][AT_PS]
  const int seq = tiles[2 * blockIdx.x], r0 = tiles[2 * blockIdx.x + 1];
  const int qbeg = cu_q[seq], qlen = cu_q[seq + 1] - qbeg;
  const int nrow = min(16, qlen - r0);
  const int row0 = qbeg + r0;
  const int pos0 = pos[row0];                // positions of a portion are consecutive
  const int last = pos0 + nrow - 1;
  const int* tab = bt + (long)seq * maxb;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, fr = lane & 15, fq = lane >> 4;
  const int rep = H / G, KC = Dk / 32;
  // sink: a logit without key or value, counted once per (head, query) -- by the first key split
  const bool sunk = sink != nullptr && blockIdx.y == 0;
  for (int e = tid; e < H * 16; e += NW * 64) { mrun[e] = sunk ? sink[e >> 4] : -INFINITY; lrun[e] = sunk ? 1.f : 0.f; }
  f32x4 o[HPW][NDV];
#pragma unroll
  for (int a = 0; a < HPW; ++a)
#pragma unroll
    for (int b = 0; b < NDV; ++b) o[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  // a wave owns HPW consecutive heads: heads of one kv group share their K and V fragments.
  // Q fragments (A operand: row fr, k = 32 kc + 8 fq) stay in registers for the whole key loop
  // where the register file allows (one wave per SIMD); keys wider than 128 are re-read.
  constexpr bool QREG = HPW * NDV <= 8 || (NW == 8 && HPW == 2);
  const int h0 = wave * HPW;
  bf16x8 qa[QREG ? HPW : 1][4];
  if constexpr (QREG) {
#pragma unroll
    for (int hi = 0; hi < HPW; ++hi)
#pragma unroll
      for (int kc2 = 0; kc2 < 4; ++kc2) {
        bf16x8 v = {};
        if (h0 + hi < H && kc2 < KC)
          v = *(const bf16x8*)(q + ((long)(row0 + min(fr, nrow - 1)) * H + h0 + hi) * Dk + 32 * kc2 + 8 * fq);
        qa[hi][kc2] = v;
      }
  }
  int lo0 = chunk > 0 ? (pos0 / chunk) * chunk : 0;
  if (window > 0) lo0 = max(lo0, pos0 - window + 1);
  __syncthreads();
  // blockIdx.y = key split: every nsplit-th key tile (decode rows: few query rows, many keys).
  // Block-table entries are read one tile ahead (K fragments) or a phase ahead (V fragments), so
  // no fragment load waits behind a dependent table load.
  const int jfirst = (lo0 / AT_KT + (int)blockIdx.y) * AT_KT;
  int nextA[2];
#pragma unroll
  for (int ns = 0; ns < 2; ++ns) {
    const int key = jfirst + 16 * ns + fr;
    nextA[ns] = key <= last ? tab[key / BS] : -1;
  }
  for (int j0 = jfirst; j0 <= last; j0 += AT_KT * nsplit) {
    int blkA[2];
#pragma unroll
    for (int ns = 0; ns < 2; ++ns) {
      blkA[ns] = nextA[ns];
      const int key = j0 + AT_KT * nsplit + 16 * ns + fr;
      nextA[ns] = key <= last ? tab[key / BS] : -1;
    }
    const int key8 = j0 + 8 * fq;
    int blk8 = -1, off8 = 0;
    if (key8 <= last) { blk8 = tab[key8 / BS]; off8 = key8 % BS; }
    // ---- A: raw scores
    for (int kb0 = 0; kb0 < KC; kb0 += 4) {      // key widths beyond 128: 128 at a time
      // 16 keys at a time: this wave's heads against their group's K fragments (B operand: key fr,
      // k = 32 kc + 8 fq), reloaded only when the kv group changes from one head to the next
#pragma unroll 1
      for (int ns = 0; ns < 2; ++ns) {
        bf16x8 kf[4];
        int gprev = -1;
        const int key = j0 + 16 * ns + fr;
        auto head = [&](int h, auto&& qfrag) {
          const int g = h / rep;
          if (g != gprev) {
            gprev = g;
            const bf16* kp = nullptr;
            const int blk = ns ? blkA[1] : blkA[0];
            if (blk >= 0) kp = kc + (((long)blk * G + g) * BS + key % BS) * Dk;
#pragma unroll
            for (int kc2 = 0; kc2 < 4; ++kc2) {
              bf16x8 v = {};
              if (kp && kb0 + kc2 < KC) v = *(const bf16x8*)(kp + 32 * (kb0 + kc2) + 8 * fq);
              kf[kc2] = v;
            }
          }
          const float slope = slopes ? slopes[h] : 0.f;
          const bf16* qp = q + ((long)(row0 + min(fr, nrow - 1)) * H + h) * Dk;
          f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kc2 = 0; kc2 < 4; ++kc2) {
            if (kb0 + kc2 < KC) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag(qp, kc2), kf[kc2], a, 0, 0, 0);
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int qr = 4 * fq + i;
            if (qr >= nrow) continue;
            float* sp = s1 + (h * 16 + qr) * AT_SS + 16 * ns + fr;
            if (kb0 > 0) a[i] += *sp;              // partial dot products of the earlier 128 columns
            if (kb0 + 4 < KC) { *sp = a[i]; continue; }
            const int qpos = pos0 + qr;
            float sc = a[i] * scale;
            if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
            sc -= slope * (float)(qpos - key);
            if (dbias) sc += dbias[(long)min(max(qpos - key, 0), nbias - 1) * H + h];
            if (key > qpos || qr >= nrow) sc = 0.f;   // hidden below; finite for the mix
            *sp = sc;
          }
        };
        if constexpr (QREG) {
#pragma unroll
          for (int hi = 0; hi < HPW; ++hi)
            if (h0 + hi < H)
              head(h0 + hi, [&](const bf16* qp, int kc2) {
                return kb0 == 0 ? qa[hi][kc2] : *(const bf16x8*)(qp + 32 * (kb0 + kc2) + 8 * fq);
              });
        } else {
#pragma unroll 1
          for (int hi = 0; hi < HPW; ++hi)
            if (h0 + hi < H)
              head(h0 + hi, [&](const bf16* qp, int kc2) { return *(const bf16x8*)(qp + 32 * (kb0 + kc2) + 8 * fq); });
        }
      }
    }
    __syncthreads();
    // ---- B: head mix (fp32 MFMA) + visibility, in place
    for (int cb = wave; cb < 2 * nrow; cb += NW) {   // (query row, 16 keys) column blocks of the live rows
      const int qr = cb >> 1, kk = (cb & 1) * 16 + fr;
      f32x4 acc[4];
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
      const int MB = (H + 15) >> 4;
      if (talk) {
        for (int ks = 0; ks < (H + 3) >> 2; ++ks) {
          const int g = 4 * ks + fq;
          const float b = g < H ? s1[(g * 16 + qr) * AT_SS + kk] : 0.f;
#pragma unroll
          for (int mb = 0; mb < 4; ++mb) {
            if (mb < MB) {
              const int m = 16 * mb + fr;
              const float a = (m < H && g < H) ? talk[m * H + g] : 0.f;
              acc[mb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[mb], 0, 0, 0);
            }
          }
        }
      }
      const int key = j0 + kk, qpos = pos0 + qr;
      int lo = chunk > 0 ? (qpos / chunk) * chunk : 0;
      if (window > 0) lo = max(lo, qpos - window + 1);
      const bool vis = qr < nrow && key <= qpos && key >= lo;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
        if (mb < MB) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int h = 16 * mb + 4 * fq + i;
            if (h < H) {
              float* p = s1 + (h * 16 + qr) * AT_SS + kk;
              const float v = talk ? acc[mb][i] : *p;
              *p = vis ? v : -INFINITY;
            }
          }
        }
      }
    }
    __syncthreads();
    // V fragments of this tile, requested before the softmax where the wave's heads share one kv
    // group and the registers are there: the loads fly while phase C runs
    constexpr bool VPRE = HPW * NDV <= 16;
    const bool one_group = h0 < H && (h0 / rep) == ((min(h0 + HPW, H) - 1) / rep);
    bf16x8 vpre[VPRE ? NDV : 1];
    if constexpr (VPRE) {
      if (one_group) {
        const int g = h0 / rep;
#pragma unroll
        for (int nd = 0; nd < NDV; ++nd) {
          const int d = 16 * nd + fr;
          bf16x8 v = {};
          if (blk8 >= 0 && d < Dv) v = *(const bf16x8*)(vc + (((((long)blk8 * G + g) * (BS >> 3) + (off8 >> 3)) * Dv) + d) * 8);
          vpre[nd] = v;
        }
      }
    }
    // ---- C: online softmax, a thread per (head, query) row
    for (int r = tid; r < H * 16; r += NW * 64) {
      if ((r & 15) >= nrow) continue;            // rows past the portion's end (decode: 15 of 16)
      const float* sr = s1 + r * AT_SS;
      float mx = -INFINITY;
#pragma unroll 8
      for (int k = 0; k < AT_KT; ++k) mx = fmaxf(mx, sr[k]);
      const float mo = mrun[r], mn = fmaxf(mo, mx);
      float sum = 0.f;
      bf16* pr = pb + r * AT_PS;
#pragma unroll 8
      for (int k = 0; k < AT_KT; ++k) {
        const float p = (sr[k] == -INFINITY) ? 0.f : __expf(sr[k] - mn);
        sum += p;
        pr[k] = (bf16)p;
      }
      const float a = (mo == -INFINITY) ? 0.f : __expf(mo - mn);
      alpha[r] = a;
      lrun[r] = lrun[r] * a + sum;
      mrun[r] = mn;
    }
    __syncthreads();
    // ---- D: O += P V; a V fragment (B operand: channel fr, keys 8 fq ..) serves every head of its group
    {
      bf16x8 pa[HPW];
#pragma unroll
      for (int hi = 0; hi < HPW; ++hi) {
        const int h = h0 + hi;
        bf16x8 v = {};
        if (h < H) {
          v = *(const bf16x8*)(pb + (h * 16 + fr) * AT_PS + 8 * fq);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float al = alpha[h * 16 + 4 * fq + i];
#pragma unroll
            for (int nd = 0; nd < NDV; ++nd) o[hi][nd][i] *= al;
          }
        }
        pa[hi] = v;
      }
#pragma unroll
      for (int nd = 0; nd < NDV; ++nd) {
        const int d = 16 * nd + fr;
        bf16x8 vb = {};
        int gprev = -1;
#pragma unroll
        for (int hi = 0; hi < HPW; ++hi) {
          const int h = h0 + hi;
          if (h >= H) continue;
          const int g = h / rep;
          if (g != gprev) {
            gprev = g;
            bool have = false;
            if constexpr (VPRE) {
              if (one_group) { vb = vpre[nd]; have = true; }
            }
            if (!have) {
              vb = bf16x8{};
              if (blk8 >= 0 && d < Dv)
                vb = *(const bf16x8*)(vc + (((((long)blk8 * G + g) * (BS >> 3) + (off8 >> 3)) * Dv) + d) * 8);
            }
          }
          o[hi][nd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[hi], vb, o[hi][nd], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int hi = 0; hi < HPW; ++hi) {
    const int h = h0 + hi;
    if (h >= H) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int qr = 4 * fq + i;
      if (qr >= nrow) continue;
      if (nsplit > 1) {   // unnormalised partial result of this key split; attn_mix_merge_kernel finishes
        const long base = ((long)(row0 + qr) * H + h) * nsplit + blockIdx.y;
        if (fr == 0) {
          part_ml[2 * base] = mrun[h * 16 + qr];
          part_ml[2 * base + 1] = lrun[h * 16 + qr];
        }
#pragma unroll
        for (int nd = 0; nd < NDV; ++nd) {
          const int d = 16 * nd + fr;
          if (d < Dv) part_o[base * Dv + d] = o[hi][nd][i];
        }
        continue;
      }
      const float l = lrun[h * 16 + qr];
      float f = l > 0.f ? 1.f / l : 0.f;
      if (gate) f *= 1.f / (1.f + __expf(-(float)gate[(long)(row0 + qr) * ldg + h]));
#pragma unroll
      for (int nd = 0; nd < NDV; ++nd) {
        const int d = 16 * nd + fr;
        if (d < Dv) out[((long)(row0 + qr) * H + h) * Dv + d] = (bf16)(o[hi][nd][i] * f);
      }
    }
  }
}

// out[row][h][d] = gate * sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M) over the key splits
__global__ __launch_bounds__(128) void attn_mix_merge_kernel(const float* __restrict__ part_o,
                                                             const float* __restrict__ part_ml, int nsplit, int H, int Dv,
                                                             const bf16* __restrict__ gate, int ldg,
                                                             bf16* __restrict__ out) {
  const int row = blockIdx.x, h = blockIdx.y;
  const long base = ((long)row * H + h) * nsplit;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_ml[2 * (base + s)]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float m = part_ml[2 * (base + s)];
    if (m != -INFINITY) L = fmaf(part_ml[2 * (base + s) + 1], __expf(m - M), L);
  }
  float f = L > 0.f ? 1.f / L : 0.f;
  if (gate) f *= 1.f / (1.f + __expf(-(float)gate[(long)row * ldg + h]));
  for (int d = threadIdx.x; d < Dv; d += 128) {
    float acc = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float m = part_ml[2 * (base + s)];
      if (m != -INFINITY) acc = fmaf(part_o[(base + s) * Dv + d], __expf(m - M), acc);
    }
    out[((long)row * H + h) * Dv + d] = (bf16)(acc * f);
  }
}

template <int NW, int HPW, int NDV>
static int launch_tile(int nsplit, void* part_o, void* part_ml, int ntiles, size_t shm, hipStream_t s, const void* q, const void* kc, const void* vc,
                       const void* tiles, const void* cu_q, const void* pos, const void* bt, int maxb, int H, int G,
                       int Dk, int Dv, int BS, float scale, float softcap, const void* slopes, const void* talk,
                       int chunk, int window, const void* gate, int ldg, void* out, const void* dbias, int nbias,
                       const void* sink) {
  auto k = attn_mix_tile_kernel<NW, HPW, NDV>;
  if (shm > 48 * 1024) (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);
  hipLaunchKernelGGL(k, dim3(ntiles, nsplit), dim3(NW * 64), shm, s, (const bf16*)q, (const bf16*)kc, (const bf16*)vc,
                     (const int*)tiles, (const int*)cu_q, (const int*)pos, (const int*)bt, maxb, H, G, Dk, Dv, BS, scale,
                     softcap, (const float*)slopes, (const float*)talk, chunk, window, (const bf16*)gate, ldg,
                     (bf16*)out, nsplit, (float*)part_o, (float*)part_ml, (const float*)dbias, nbias, (const float*)sink);
  return (int)hipGetLastError();
}

}  // namespace la

extern "C" int la_attn_mix_rows(int f32, const void* q, const void* kc, const void* vc, const void* row_seq,
                                const void* pos, const void* bt, int maxb, int T, int H, int G, int Dk, int Dv, int BS,
                                float scale, float softcap, const void* slopes, const void* talk, int chunk, int window,
                                const void* gate, int ldg, void* out, const void* dbias, int nbias, const void* sink,
                                void* stream) {
  using namespace la;
  if (T <= 0 || H <= 0 || G <= 0 || H % G || H * Dv > AM_NT * AM_MAXO || (dbias && nbias < 1)) return -1;
  const size_t shm = sizeof(float) * ((size_t)H * Dk + 2 * (size_t)H * AM_KT + 3 * (size_t)H);
  if (shm > 160 * 1024) return -2;
  hipStream_t s = (hipStream_t)stream;
  if (f32) {
    if (shm > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)attn_mix_rows_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);
    hipLaunchKernelGGL((attn_mix_rows_kernel<float>), dim3(T), dim3(AM_NT), shm, s, (const float*)q, (const float*)kc,
                       (const float*)vc, (const int*)row_seq, (const int*)pos, (const int*)bt, maxb, H, G, Dk, Dv, BS,
                       scale, softcap, (const float*)slopes, (const float*)talk, chunk, window, (const float*)gate, ldg,
                       (float*)out, (const float*)dbias, nbias, (const float*)sink);
  } else {
    if (shm > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)attn_mix_rows_kernel<bf16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shm);
    hipLaunchKernelGGL((attn_mix_rows_kernel<bf16>), dim3(T), dim3(AM_NT), shm, s, (const bf16*)q, (const bf16*)kc,
                       (const bf16*)vc, (const int*)row_seq, (const int*)pos, (const int*)bt, maxb, H, G, Dk, Dv, BS,
                       scale, softcap, (const float*)slopes, (const float*)talk, chunk, window, (const bf16*)gate, ldg,
                       (bf16*)out, (const float*)dbias, nbias, (const float*)sink);
  }
  return (int)hipGetLastError();
}

// Prompt portions (bf16): tiles [ntiles][2] = (sequence, first row of the tile within the
// sequence's portion), 16 rows per tile.  Returns 1 when the shape is outside the kernel's reach
// (the caller then uses la_attn_mix_rows): Dk % 32, Dv % 16, Dv <= 128, H <= 32, BS % 8.
// nsplit > 1 (batches of few rows with many keys, i.e. decoding): every tile's keys are dealt to
// nsplit workgroups whose partial results (part_o [rows, H, nsplit, Dv], part_ml [rows, H, nsplit, 2],
// fp32, rows = the batch rows the tiles cover) a second launch merges.
extern "C" int la_attn_mix_tiles(const void* q, const void* kc, const void* vc, const void* tiles, int ntiles,
                                 const void* cu_q, const void* pos, const void* bt, int maxb, int H, int G, int Dk,
                                 int Dv, int BS, float scale, float softcap, const void* slopes, const void* talk,
                                 int chunk, int window, const void* gate, int ldg, void* out, int nsplit, void* part_o,
                                 void* part_ml, int rows, const void* dbias, int nbias, const void* sink, void* stream) {
  using namespace la;
  if (ntiles <= 0 || H <= 0 || G <= 0 || H % G || nsplit < 1 || nsplit > 64 || (nsplit > 1 && (!part_o || !part_ml)) ||
      (dbias && nbias < 1))
    return -1;
  if ((Dk % 32) || (Dv % 16) || Dv > 128 || H > 32 || (BS & 7)) return 1;
  const size_t shm = (size_t)H * 16 * (AT_SS * 4 + 3 * 4 + AT_PS * 2);
  if (shm > 150 * 1024) return 1;
  hipStream_t s = (hipStream_t)stream;
  // 8 waves from 9 heads on: fewer heads (accumulator registers) per wave, more waves to hide latency
  const int nw = H > 8 ? 8 : 4, hpw = (H + nw - 1) / nw, ndv = Dv <= 32 ? 2 : (Dv <= 64 ? 4 : 8);
  int rc = 1;
#define LA_TILE(NW, HPW, NDV)                                                                                      \
  if (rc == 1 && nw == NW && hpw <= HPW && ndv == NDV)                                                             \
    rc = launch_tile<NW, HPW, NDV>(nsplit, part_o, part_ml, ntiles, shm, s, q, kc, vc, tiles, cu_q, pos, bt, maxb, H, \
                                   G, Dk, Dv, BS, scale, softcap, slopes, talk, chunk, window, gate, ldg, out, dbias,    \
                                   nbias, sink);
  LA_TILE(4, 1, 2) LA_TILE(4, 1, 4) LA_TILE(4, 1, 8) LA_TILE(4, 2, 2) LA_TILE(4, 2, 4) LA_TILE(4, 2, 8)
  LA_TILE(8, 2, 2) LA_TILE(8, 2, 4) LA_TILE(8, 2, 8) LA_TILE(8, 4, 2) LA_TILE(8, 4, 4) LA_TILE(8, 4, 8)
#undef LA_TILE
  if (rc == 0 && nsplit > 1) {
    hipLaunchKernelGGL(attn_mix_merge_kernel, dim3(rows, H), dim3(128), 0, s, (const float*)part_o, (const float*)part_ml,
                       nsplit, H, Dv, (const bf16*)gate, ldg, (bf16*)out);
    rc = (int)hipGetLastError();
  }
  return rc;
}
