// Mixture-of-experts pieces for dense (bf16 / fp32) expert weights of any width:
//   * a router with sigmoid scores, an optional selection-only correction and normalised weights,
//     or with biased logits and the softmax over the chosen logits as weights;
//   * the routed experts of small batches as (token, expert) pair GEMVs: gate|up with the SiLU
//     gating fused, then the down projection with the weighted top-k combine fused, no atomics.
// Larger batches group rows by expert and run library GEMMs (the caller's choice).
#include "common.h"

namespace la {

// One wave per token: z_e = router[e] . x (fp32).
// mode 0: s = sigmoid(z); the `topk` largest s + corr are chosen (ties: lowest expert id), their
//         weights are s / (sum of the chosen s + 1e-20).
// mode 1: s = z + corr (a bias that counts in the weights too); the `topk` largest s are chosen,
//         their weights are the softmax over the chosen s.
template <typename AT>
__global__ __launch_bounds__(256) void router_topk_kernel(const AT* __restrict__ x, long ldx,
                                                          const float* __restrict__ router,
                                                          const float* __restrict__ corr, int E, int D, int T,
                                                          int topk, int renorm, int mode, int* __restrict__ ids,
                                                          float* __restrict__ wts) {
  __shared__ float sc[4][256];
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + w;
  const bool live = t < T;
  const AT* xr = x + (long)(live ? t : 0) * ldx;
  // 8 experts at a time: x is read once per pass and the 8 router rows give independent loads
  for (int e0 = 0; e0 < E; e0 += 8) {
    float a[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] = 0.f;
    if ((D & 3) == 0) {
      for (int d = lane * 4; d < D; d += 256) {
        const float x0 = (float)xr[d], x1 = (float)xr[d + 1], x2 = (float)xr[d + 2], x3 = (float)xr[d + 3];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          if (e0 + k < E) {
            const float4 r = *(const float4*)(router + (long)(e0 + k) * D + d);
            a[k] = fmaf(r.x, x0, fmaf(r.y, x1, fmaf(r.z, x2, fmaf(r.w, x3, a[k]))));
          }
        }
      }
    } else {
      for (int d = lane; d < D; d += 64) {
        const float xv = (float)xr[d];
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (e0 + k < E) a[k] = fmaf(router[(long)(e0 + k) * D + d], xv, a[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float v = wave_sum(a[k]);
      if (lane == 0 && e0 + k < E) sc[w][e0 + k] = mode ? v + (corr ? corr[e0 + k] : 0.f) : 1.f / (1.f + __expf(-v));
    }
  }
  __syncthreads();
  float sum = 0.f, my_s = 0.f, top0 = 0.f;
  int my_id = 0;
  uint32_t taken = 0;   // bit i: this lane's expert e = lane + 64 * i is already chosen
  for (int k = 0; k < topk; ++k) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = 0; i < 4; ++i) {
      const int e = lane + 64 * i;
      if (e < E && !((taken >> i) & 1u)) {
        const float c = sc[w][e] + ((corr && !mode) ? corr[e] : 0.f);
        if (c > best || (c == best && e < bi)) { best = c; bi = e; }
      }
    }
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if ((bi & 63) == lane) taken |= 1u << (bi >> 6);
    float s = sc[w][bi];
    if (mode) {           // softmax over the chosen logits: the first chosen one is the largest
      if (k == 0) top0 = s;
      s = expf(s - top0);
    }
    sum += s;
    if (lane == k) { my_s = s; my_id = bi; }
  }
  if (live && lane < topk) {
    ids[(long)t * topk + lane] = my_id;
    wts[(long)t * topk + lane] = (renorm || mode) ? my_s / (sum + 1e-20f) : my_s;
  }
}

// h[p][f] = silu(Wg[e_p][f] . x[t_p]) * (Wu[e_p][f] . x[t_p]),  p = t * topk + slot; a wave per (p, f).
// clamp: g = min(Wg x, limit), u = clamp(Wu x, -limit, limit), h = g sigmoid(slope g) (u + 1) instead.
template <typename AT, typename WT>
__global__ __launch_bounds__(256) void moe_pair_glu_kernel(const AT* __restrict__ x, const WT* __restrict__ wg,
                                                           const WT* __restrict__ wu, const int* __restrict__ ids,
                                                           int topk, int D, int F, int E, AT* __restrict__ h, int clamp,
                                                           float limit, float slope) {
  const int p = blockIdx.y;
  const int f = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (f >= F) return;
  const int e = ids[p];
  if (e < 0 || e >= E) { if (lane == 0) h[(long)p * F + f] = (AT)0.f; return; }
  const AT* xr = x + (long)(p / topk) * D;
  const WT* g = wg + ((long)e * F + f) * D;
  const WT* u = wu + ((long)e * F + f) * D;
  float a = 0.f, b = 0.f;
  for (int d = lane; d < D; d += 64) {
    const float xv = (float)xr[d];
    a = fmaf((float)g[d], xv, a);
    b = fmaf((float)u[d], xv, b);
  }
  a = wave_sum(a);
  b = wave_sum(b);
  if (lane == 0) {
    float v;
    if (clamp) {
      const float g2 = fminf(a, limit), u2 = fminf(fmaxf(b, -limit), limit);
      v = g2 / (1.f + expf(-slope * g2)) * (u2 + 1.f);
    } else {
      v = silu(a) * b;
    }
    h[(long)p * F + f] = (AT)v;
  }
}

// y[t][d] = sum_slot w[p] * (Wd[e_p][d] . h[p]); a wave per (t, d), slots in order (deterministic)
template <typename AT, typename WT>
__global__ __launch_bounds__(256) void moe_pair_down_kernel(const AT* __restrict__ h, const WT* __restrict__ wd,
                                                            const int* __restrict__ ids, const float* __restrict__ wts,
                                                            int topk, int D, int F, int E, float* __restrict__ y) {
  const int t = blockIdx.y;
  const int d = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (d >= D) return;
  float acc = 0.f;
  for (int k = 0; k < topk; ++k) {
    const int p = t * topk + k, e = ids[p];
    if (e < 0 || e >= E) continue;
    const WT* wr = wd + ((long)e * D + d) * F;
    const AT* hr = h + (long)p * F;
    float a = 0.f;
    for (int f = lane; f < F; f += 64) a = fmaf((float)wr[f], (float)hr[f], a);
    acc = fmaf(wts[p], wave_sum(a), acc);
  }
  if (lane == 0) y[(long)t * D + d] = acc;
}

}  // namespace la

extern "C" int la_router_topk(int f32, int mode, const void* x, long ldx, const void* router, const void* corr, int E,
                              int D, int T, int topk, int renorm, void* ids, void* wts, void* stream) {
  using namespace la;
  if (E < 1 || E > 256 || topk < 1 || topk > E || topk > 64 || T <= 0 || mode < 0 || mode > 1) return -1;
  dim3 grid((T + 3) / 4);
  if (f32)
    hipLaunchKernelGGL((router_topk_kernel<float>), grid, dim3(256), 0, (hipStream_t)stream, (const float*)x, ldx,
                       (const float*)router, (const float*)corr, E, D, T, topk, renorm, mode, (int*)ids, (float*)wts);
  else
    hipLaunchKernelGGL((router_topk_kernel<bf16>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16*)x, ldx,
                       (const float*)router, (const float*)corr, E, D, T, topk, renorm, mode, (int*)ids, (float*)wts);
  return (int)hipGetLastError();
}

extern "C" int la_router_sigmoid(int f32, const void* x, long ldx, const void* router, const void* corr, int E, int D,
                                 int T, int topk, int renorm, void* ids, void* wts, void* stream) {
  return la_router_topk(f32, 0, x, ldx, router, corr, E, D, T, topk, renorm, ids, wts, stream);
}

// f32: activations and weights fp32 (else both bf16).  x [T, D], wg / wu [E, F, D], wd [E, D, F],
// ids [T * topk], wts [T * topk] -> h [T * topk, F] (scratch, activation type), y [T, D] fp32.
extern "C" int la_moe_pairs(int f32, const void* x, const void* wg, const void* wu, const void* wd, const void* ids,
                            const void* wts, int T, int topk, int D, int F, int E, void* h, void* y, int clamp, float limit,
                            float slope, void* stream) {
  using namespace la;
  if (T <= 0 || topk < 1 || D < 1 || F < 1) return -1;
  const int P = T * topk;
  if (P > 65535 || T > 65535) return -2;
  dim3 g1((F + 3) / 4, P), g2((D + 3) / 4, T);
  hipStream_t s = (hipStream_t)stream;
  if (f32) {
    hipLaunchKernelGGL((moe_pair_glu_kernel<float, float>), g1, dim3(256), 0, s, (const float*)x, (const float*)wg,
                       (const float*)wu, (const int*)ids, topk, D, F, E, (float*)h, clamp, limit, slope);
    hipLaunchKernelGGL((moe_pair_down_kernel<float, float>), g2, dim3(256), 0, s, (const float*)h, (const float*)wd,
                       (const int*)ids, (const float*)wts, topk, D, F, E, (float*)y);
  } else {
    hipLaunchKernelGGL((moe_pair_glu_kernel<bf16, bf16>), g1, dim3(256), 0, s, (const bf16*)x, (const bf16*)wg,
                       (const bf16*)wu, (const int*)ids, topk, D, F, E, (bf16*)h, clamp, limit, slope);
    hipLaunchKernelGGL((moe_pair_down_kernel<bf16, bf16>), g2, dim3(256), 0, s, (const bf16*)h, (const bf16*)wd,
                       (const int*)ids, (const float*)wts, topk, D, F, E, (float*)y);
  }
  return (int)hipGetLastError();
}
