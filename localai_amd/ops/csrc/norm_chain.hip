// Sublayer boundaries of a post-normed fp32 residual stream, and the small elementwise steps of
// layer-list designs that sit between two library GEMMs.
//
//   norm_chain:  res <- (replace ? 0 : res) + post(branch) + add_vec;  out = pre(res)
//       post:  none | dyt: tanh(alpha y) * w + b | rms: y / sqrt(mean(y^2) + eps) * w
//              | ln: (y - mean) / sqrt(mean((y - mean)^2) + eps) * w  (layer norm, no bias)
//       pre:   none | dyt | cast (the stream itself in the output type) | ln (eps in the alpha slot)
//     one launch where a pre-normed stream has "add + norm": the branch's own norm, the residual
//     add and the next sublayer's input norm.  A workgroup per row; the rms variant reads the
//     branch row twice (second time from cache) instead of holding it in registers, so any width runs.
//   add_group_norm:  res += branch;  out = res normed in equal consecutive groups (each / its own rms) times w:
//     the boundary of a pre-normed fp32 stream whose norm works on groups
//   poly_norm_act:   y = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e over a row
//   sigmoid_mul:     x * sigmoid(gate), the gate being columns of a wider row
//   glu_clamp:   g = min(gate, limit), u = clamp(up, -limit, limit), y = g sigmoid(slope g) (u + 1)
//   side_gate:   gelu_tanh(z[t][c]) * table[tok[t]][col0 + c]
//
// Sources are GEMM results as the framework hands them on: fp32 split-K slabs [S][T][N] (summed
// here), or one bf16 / fp32 matrix.  All arithmetic is fp32; outputs bf16 or fp32.
#include "common.h"

namespace la {

struct RowSrc {
  const void* p;
  int f32;
  long slab;
  int S;
};

LA_DEV float src_at(const RowSrc& s, long idx) {
  if (s.f32) {
    const float* f = (const float*)s.p;
    float a = f[idx];
    for (int k = 1; k < s.S; ++k) a += f[idx + k * s.slab];
    return a;
  }
  return (float)((const bf16*)s.p)[idx];
}

LA_DEV void put(void* out, int out_f32, long idx, float v) {
  if (out_f32) ((float*)out)[idx] = v;
  else ((bf16*)out)[idx] = (bf16)v;
}

enum { NC_NONE = 0, NC_DYT = 1, NC_RMS = 2, NC_CAST = 3, NC_LN = 4 };
constexpr int NC_NT = 256;

__global__ __launch_bounds__(NC_NT) void norm_chain_kernel(float* __restrict__ res, int D, RowSrc src, int has_src,
                                                           int post, float pa, const float* __restrict__ pw,
                                                           const float* __restrict__ pb, float eps,
                                                           const float* __restrict__ addv, int replace, int pre,
                                                           float qa, const float* __restrict__ qw,
                                                           const float* __restrict__ qb, void* __restrict__ out,
                                                           int out_f32) {
  __shared__ float red[NC_NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x;
  const long base = (long)t * D;
  float inv = 1.f, mean = 0.f;
  if (has_src && (post == NC_RMS || post == NC_LN)) {
    if (post == NC_LN) {
      float sm = 0.f;
      for (int c = tid; c < D; c += NC_NT) sm += src_at(src, base + c);
      mean = block_sum<NC_NT>(sm, red) / (float)D;
    }
    float ss = 0.f;
    for (int c = tid; c < D; c += NC_NT) {
      const float y = src_at(src, base + c) - mean;
      ss = fmaf(y, y, ss);
    }
    ss = block_sum<NC_NT>(ss, red);
    inv = 1.f / sqrtf(ss / (float)D + eps);
  }
  for (int c = tid; c < D; c += NC_NT) {
    float x = res[base + c];
    if (has_src) {
      float y = src_at(src, base + c);
      if (post == NC_DYT) y = fmaf(tanhf(pa * y), pw[c], pb[c]);
      else if (post == NC_RMS || post == NC_LN) y = (y - mean) * inv * pw[c];
      if (addv) y += addv[c];
      x = replace ? y : x + y;
      res[base + c] = x;
    }
    if (pre == NC_DYT) put(out, out_f32, base + c, fmaf(tanhf(qa * x), qw[c], qb[c]));
    else if (pre == NC_CAST) put(out, out_f32, base + c, x);
  }
  if (pre == NC_LN) {   // layer norm of the updated row: every thread re-reads the columns it wrote
    float sm = 0.f;
    for (int c = tid; c < D; c += NC_NT) sm += res[base + c];
    const float m2 = block_sum<NC_NT>(sm, red) / (float)D;
    float ss = 0.f;
    for (int c = tid; c < D; c += NC_NT) {
      const float d = res[base + c] - m2;
      ss = fmaf(d, d, ss);
    }
    const float inv2 = 1.f / sqrtf(block_sum<NC_NT>(ss, red) / (float)D + qa);
    for (int c = tid; c < D; c += NC_NT) put(out, out_f32, base + c, (res[base + c] - m2) * inv2 * qw[c]);
  }
}

// widths that are a multiple of 4 with one-matrix sources: 4 columns per thread, 16-byte accesses to the stream
__global__ __launch_bounds__(NC_NT) void norm_chain4_kernel(float* __restrict__ res, int D, const void* __restrict__ sp,
                                                            int src_f32, int has_src, int post, float pa,
                                                            const float* __restrict__ pw, const float* __restrict__ pb,
                                                            float eps, const float* __restrict__ addv, int replace,
                                                            int pre, float qa, const float* __restrict__ qw,
                                                            const float* __restrict__ qb, void* __restrict__ out,
                                                            int out_f32) {
  __shared__ float red[NC_NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x;
  const long base = (long)t * D;
  auto load = [&](int c, float* y) {
    if (src_f32) {
      const float4 v = *(const float4*)((const float*)sp + base + c);
      y[0] = v.x; y[1] = v.y; y[2] = v.z; y[3] = v.w;
    } else {
      const bf16x4 v = *(const bf16x4*)((const bf16*)sp + base + c);
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] = (float)v[j];
    }
  };
  float inv = 1.f, mean = 0.f;
  if (has_src && (post == NC_RMS || post == NC_LN)) {
    if (post == NC_LN) {
      float sm = 0.f;
      for (int c = tid * 4; c < D; c += NC_NT * 4) {
        float y[4];
        load(c, y);
        sm += (y[0] + y[1]) + (y[2] + y[3]);
      }
      mean = block_sum<NC_NT>(sm, red) / (float)D;
    }
    float ss = 0.f;
    for (int c = tid * 4; c < D; c += NC_NT * 4) {
      float y[4];
      load(c, y);
#pragma unroll
      for (int j = 0; j < 4; ++j) ss = fmaf(y[j] - mean, y[j] - mean, ss);
    }
    ss = block_sum<NC_NT>(ss, red);
    inv = 1.f / sqrtf(ss / (float)D + eps);
  }
  for (int c = tid * 4; c < D; c += NC_NT * 4) {
    const float4 xv = *(const float4*)(res + base + c);
    float x[4] = {xv.x, xv.y, xv.z, xv.w};
    if (has_src) {
      float y[4];
      load(c, y);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (post == NC_DYT) y[j] = fmaf(tanhf(pa * y[j]), pw[c + j], pb[c + j]);
        else if (post == NC_RMS || post == NC_LN) y[j] = (y[j] - mean) * inv * pw[c + j];
        if (addv) y[j] += addv[c + j];
        x[j] = replace ? y[j] : x[j] + y[j];
      }
      *(float4*)(res + base + c) = make_float4(x[0], x[1], x[2], x[3]);
    }
    if (pre == NC_DYT || pre == NC_CAST) {
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = pre == NC_DYT ? fmaf(tanhf(qa * x[j]), qw[c + j], qb[c + j]) : x[j];
      if (out_f32) *(float4*)((float*)out + base + c) = make_float4(o[0], o[1], o[2], o[3]);
      else {
        bf16x4 ob = {(bf16)o[0], (bf16)o[1], (bf16)o[2], (bf16)o[3]};
        *(bf16x4*)((bf16*)out + base + c) = ob;
      }
    }
  }
  if (pre == NC_LN) {   // layer norm of the updated row: every thread re-reads the columns it wrote
    float sm = 0.f;
    for (int c = tid * 4; c < D; c += NC_NT * 4) {
      const float4 v = *(const float4*)(res + base + c);
      sm += (v.x + v.y) + (v.z + v.w);
    }
    const float m2 = block_sum<NC_NT>(sm, red) / (float)D;
    float ss = 0.f;
    for (int c = tid * 4; c < D; c += NC_NT * 4) {
      const float4 v = *(const float4*)(res + base + c);
      ss = fmaf(v.x - m2, v.x - m2, fmaf(v.y - m2, v.y - m2, fmaf(v.z - m2, v.z - m2, fmaf(v.w - m2, v.w - m2, ss))));
    }
    const float inv2 = 1.f / sqrtf(block_sum<NC_NT>(ss, red) / (float)D + qa);
    for (int c = tid * 4; c < D; c += NC_NT * 4) {
      const float4 v = *(const float4*)(res + base + c);
      const float o[4] = {(v.x - m2) * inv2 * qw[c], (v.y - m2) * inv2 * qw[c + 1], (v.z - m2) * inv2 * qw[c + 2],
                          (v.w - m2) * inv2 * qw[c + 3]};
      if (out_f32) *(float4*)((float*)out + base + c) = make_float4(o[0], o[1], o[2], o[3]);
      else {
        bf16x4 ob = {(bf16)o[0], (bf16)o[1], (bf16)o[2], (bf16)o[3]};
        *(bf16x4*)((bf16*)out + base + c) = ob;
      }
    }
  }
}

__global__ __launch_bounds__(256) void glu_clamp_kernel(RowSrc src, int F, long total, float limit, float slope,
                                                        void* __restrict__ out, int out_f32) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const long t = e / F;
  const int c = (int)(e - t * F);
  const float g = fminf(src_at(src, t * 2 * F + c), limit);
  const float u = fminf(fmaxf(src_at(src, t * 2 * F + F + c), -limit), limit);
  put(out, out_f32, e, g / (1.f + expf(-slope * g)) * (u + 1.f));
}

// one bf16 matrix source, F % 8 == 0: 8 columns per thread, 16-byte loads and stores
__global__ __launch_bounds__(256) void glu_clamp8_kernel(const bf16* __restrict__ src, int F, float limit, float slope,
                                                         bf16* __restrict__ out) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= F) return;
  const bf16x8 gv = *(const bf16x8*)(src + (long)t * 2 * F + c);
  const bf16x8 uv = *(const bf16x8*)(src + (long)t * 2 * F + F + c);
  bf16x8 ob;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float g = fminf((float)gv[j], limit);
    const float u = fminf(fmaxf((float)uv[j], -limit), limit);
    ob[j] = (bf16)(g / (1.f + __expf(-slope * g)) * (u + 1.f));
  }
  *(bf16x8*)(out + (long)t * F + c) = ob;
}

LA_DEV float gelu_tanh_f(float x) { return 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x))); }

__global__ __launch_bounds__(256) void side_gate_kernel(RowSrc src, int n, long total, const int* __restrict__ tok,
                                                        const bf16* __restrict__ table, int ldt, int col0,
                                                        void* __restrict__ out, int out_f32) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const long t = e / n;
  const int c = (int)(e - t * n);
  const float emb = (float)table[(long)tok[t] * ldt + col0 + c];
  put(out, out_f32, e, gelu_tanh_f(src_at(src, e)) * emb);
}

// Pre-normed streams whose norm works on groups:  res += branch;  out = res, each of `groups` equal
// consecutive parts divided by its own sqrt(mean(part^2) + eps), times w.  A workgroup per row; after
// the add every wave takes whole groups (group g -> wave g mod 4), so a group's statistics need no
// workgroup-wide reduction; the row is re-read from cache.
__global__ __launch_bounds__(NC_NT) void add_group_norm_kernel(float* __restrict__ res, int D, RowSrc src, int has_src,
                                                               const float* __restrict__ w, float eps, int groups,
                                                               void* __restrict__ out, int out_f32) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const long base = (long)t * D;
  if (has_src) {
    for (int c = tid; c < D; c += NC_NT) res[base + c] += src_at(src, base + c);
    __syncthreads();
  }
  const int gs = D / groups, wave = tid >> 6, lane = tid & 63;
  for (int g = wave; g < groups; g += NC_NT / 64) {
    const float* row = res + base + (long)g * gs;
    float ss = 0.f;
    for (int c = lane; c < gs; c += 64) ss = fmaf(row[c], row[c], ss);
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)gs + eps);
    for (int c = lane; c < gs; c += 64) put(out, out_f32, base + (long)g * gs + c, row[c] * inv * w[g * gs + c]);
  }
}

// one group and few groups of wide rows: the whole workgroup per group (block reductions)
__global__ __launch_bounds__(NC_NT) void add_group_norm_wide_kernel(float* __restrict__ res, int D, RowSrc src, int has_src,
                                                                    const float* __restrict__ w, float eps, int groups,
                                                                    void* __restrict__ out, int out_f32) {
  __shared__ float red[NC_NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x;
  const long base = (long)t * D;
  const int gs = D / groups;
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    for (int c = g * gs + tid; c < (g + 1) * gs; c += NC_NT) {
      float x = res[base + c];
      if (has_src) {
        x += src_at(src, base + c);
        res[base + c] = x;
      }
      ss = fmaf(x, x, ss);
    }
    const float inv = 1.f / sqrtf(block_sum<NC_NT>(ss, red) / (float)gs + eps);
    for (int c = g * gs + tid; c < (g + 1) * gs; c += NC_NT) put(out, out_f32, base + c, res[base + c] * inv * w[c]);
  }
}

// y = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e over a row of F values (rms with eps inside
// the root): a workgroup per row, one pass for the three sums of even powers, one for the outputs
__global__ __launch_bounds__(NC_NT) void poly_norm_act_kernel(RowSrc src, int F, const float* __restrict__ coef, float eps,
                                                              void* __restrict__ out, int out_f32) {
  __shared__ float red[NC_NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x;
  const long base = (long)t * F;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int c = tid; c < F; c += NC_NT) {
    const float z = src_at(src, base + c), z2 = z * z;
    s2 += z2;
    s4 = fmaf(z2, z2, s4);
    s6 = fmaf(z2 * z2, z2, s6);
  }
  s2 = block_sum<NC_NT>(s2, red);
  s4 = block_sum<NC_NT>(s4, red);
  s6 = block_sum<NC_NT>(s6, red);
  const float i1 = coef[0] / sqrtf(s2 / (float)F + eps), i2 = coef[1] / sqrtf(s4 / (float)F + eps),
              i3 = coef[2] / sqrtf(s6 / (float)F + eps), e = coef[3];
  for (int c = tid; c < F; c += NC_NT) {
    const float z = src_at(src, base + c);
    put(out, out_f32, base + c, fmaf(z, i1, fmaf(z * z, i2, fmaf(z * z * z, i3, e))));
  }
}

// The same for one bf16 matrix with F % 8 == 0 and F <= 16384: a thread keeps its columns (up to 8 vectors
// of 8) in registers between the two passes, 16-byte loads and stores, the row is read once.
constexpr int PN_MAXV = 8;
__global__ __launch_bounds__(NC_NT) void poly_norm_act8_kernel(const bf16* __restrict__ src, int F,
                                                               const float* __restrict__ coef, float eps,
                                                               bf16* __restrict__ out) {
  __shared__ float red[NC_NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x, nv = F >> 3;
  const bf16x8* row = (const bf16x8*)(src + (long)t * F);
  bf16x8 z[PN_MAXV];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int k = 0; k < PN_MAXV; ++k) {
    const int v = tid + k * NC_NT;
    if (v < nv) {
      z[k] = row[v];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = (float)z[k][j], x2 = x * x;
        s2 += x2;
        s4 = fmaf(x2, x2, s4);
        s6 = fmaf(x2 * x2, x2, s6);
      }
    }
  }
  s2 = block_sum<NC_NT>(s2, red);
  s4 = block_sum<NC_NT>(s4, red);
  s6 = block_sum<NC_NT>(s6, red);
  const float i1 = coef[0] / sqrtf(s2 / (float)F + eps), i2 = coef[1] / sqrtf(s4 / (float)F + eps),
              i3 = coef[2] / sqrtf(s6 / (float)F + eps), e = coef[3];
  bf16x8* orow = (bf16x8*)(out + (long)t * F);
#pragma unroll
  for (int k = 0; k < PN_MAXV; ++k) {
    const int v = tid + k * NC_NT;
    if (v < nv) {
      bf16x8 y;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = (float)z[k][j];
        y[j] = (bf16)fmaf(x, i1, fmaf(x * x, i2, fmaf(x * x * x, i3, e)));
      }
      orow[v] = y;
    }
  }
}

// out = x * sigmoid(gate), gate rows with their own stride (columns of a wider projection)
__global__ __launch_bounds__(256) void sigmoid_mul_kernel(const void* __restrict__ x, int x_f32, const void* __restrict__ g,
                                                          int g_f32, long ldg, int N, long total, void* __restrict__ out,
                                                          int out_f32) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const long t = e / N;
  const int c = (int)(e - t * N);
  const float xv = x_f32 ? ((const float*)x)[e] : (float)((const bf16*)x)[e];
  const float gv = g_f32 ? ((const float*)g)[t * ldg + c] : (float)((const bf16*)g)[t * ldg + c];
  put(out, out_f32, e, xv / (1.f + expf(-gv)));
}

// bf16 operands with N % 8 == 0 and 16-byte aligned rows: 8 columns a thread
__global__ __launch_bounds__(256) void sigmoid_mul8_kernel(const bf16* __restrict__ x, const bf16* __restrict__ g, long ldg,
                                                           int N, long total8, bf16* __restrict__ out) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total8) return;
  const int nv = N >> 3;
  const long t = e / nv;
  const int c = (int)(e - t * nv) * 8;
  const bf16x8 xv = *(const bf16x8*)(x + t * N + c), gv = *(const bf16x8*)(g + t * ldg + c);
  bf16x8 y;
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = (bf16)((float)xv[j] / (1.f + expf(-(float)gv[j])));
  *(bf16x8*)(out + t * N + c) = y;
}

}  // namespace la

extern "C" int la_add_group_norm(void* res, int T, int D, const void* sp, int src_f32, long slab, int S, const void* w,
                                 float eps, int groups, void* out, int out_f32, void* stream) {
  using namespace la;
  if (T <= 0 || D <= 0 || groups < 1 || D % groups || !res || !w || !out) return -1;
  const int has = sp != nullptr;
  if (has && src_f32 && S < 1) return -4;
  RowSrc s{sp, src_f32, slab, S};
  if (groups >= 4 && D / groups <= 1024)
    hipLaunchKernelGGL(add_group_norm_kernel, dim3(T), dim3(NC_NT), 0, (hipStream_t)stream, (float*)res, D, s, has,
                       (const float*)w, eps, groups, out, out_f32);
  else
    hipLaunchKernelGGL(add_group_norm_wide_kernel, dim3(T), dim3(NC_NT), 0, (hipStream_t)stream, (float*)res, D, s, has,
                       (const float*)w, eps, groups, out, out_f32);
  return (int)hipGetLastError();
}

extern "C" int la_poly_norm_act(const void* sp, int src_f32, long slab, int S, int T, int F, const void* coef, float eps,
                                void* out, int out_f32, void* stream) {
  using namespace la;
  if (T <= 0 || F <= 0 || !sp || !coef || !out) return -1;
  if (!src_f32 && !out_f32 && (F & 7) == 0 && F <= 8 * NC_NT * PN_MAXV) {
    hipLaunchKernelGGL(poly_norm_act8_kernel, dim3(T), dim3(NC_NT), 0, (hipStream_t)stream, (const bf16*)sp, F,
                       (const float*)coef, eps, (bf16*)out);
    return (int)hipGetLastError();
  }
  RowSrc s{sp, src_f32, slab, S};
  hipLaunchKernelGGL(poly_norm_act_kernel, dim3(T), dim3(NC_NT), 0, (hipStream_t)stream, s, F, (const float*)coef, eps, out,
                     out_f32);
  return (int)hipGetLastError();
}

extern "C" int la_sigmoid_mul(const void* x, int x_f32, const void* g, int g_f32, long ldg, int T, int N, void* out,
                              int out_f32, void* stream) {
  using namespace la;
  if (T <= 0 || N <= 0 || !x || !g || !out || ldg < N) return -1;
  if (!x_f32 && !g_f32 && !out_f32 && (N & 7) == 0 && (ldg & 7) == 0 && (((uintptr_t)x | (uintptr_t)g | (uintptr_t)out) & 15) == 0) {
    const long total8 = (long)T * (N >> 3);
    hipLaunchKernelGGL(sigmoid_mul8_kernel, dim3((unsigned)((total8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const bf16*)x, (const bf16*)g, ldg, N, total8, (bf16*)out);
    return (int)hipGetLastError();
  }
  const long total = (long)T * N;
  hipLaunchKernelGGL(sigmoid_mul_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, x_f32,
                     g, g_f32, ldg, N, total, out, out_f32);
  return (int)hipGetLastError();
}

extern "C" int la_norm_chain(void* res, int T, int D, const void* sp, int src_f32, long slab, int S, int post, float pa,
                             const void* pw, const void* pb, float eps, const void* addv, int replace, int pre, float qa,
                             const void* qw, const void* qb, void* out, int out_f32, void* stream) {
  using namespace la;
  if (T <= 0 || D <= 0 || !res) return -1;
  if (post == NC_DYT && (!pw || !pb)) return -2;
  if ((post == NC_RMS || post == NC_LN) && !pw) return -2;
  if (pre == NC_DYT && (!qw || !qb)) return -2;
  if (pre == NC_LN && !qw) return -2;
  if (pre != NC_NONE && !out) return -3;
  const int has = sp != nullptr;
  if (has && src_f32 && S < 1) return -4;
  if ((D & 3) == 0 && (!has || S <= 1)) {
    hipLaunchKernelGGL(norm_chain4_kernel, dim3(T), dim3(NC_NT), 0, (hipStream_t)stream, (float*)res, D, sp, src_f32, has,
                       post, pa, (const float*)pw, (const float*)pb, eps, (const float*)addv, replace, pre, qa,
                       (const float*)qw, (const float*)qb, out, out_f32);
    return (int)hipGetLastError();
  }
  RowSrc s{sp, src_f32, slab, S};
  hipLaunchKernelGGL(norm_chain_kernel, dim3(T), dim3(NC_NT), 0, (hipStream_t)stream, (float*)res, D, s, has, post, pa,
                     (const float*)pw, (const float*)pb, eps, (const float*)addv, replace, pre, qa, (const float*)qw,
                     (const float*)qb, out, out_f32);
  return (int)hipGetLastError();
}

extern "C" int la_glu_clamp(const void* sp, int src_f32, long slab, int S, int T, int F, float limit, float slope,
                            void* out, int out_f32, void* stream) {
  using namespace la;
  if (T <= 0 || F <= 0 || !sp || !out) return -1;
  if (!src_f32 && !out_f32 && (F & 7) == 0) {
    hipLaunchKernelGGL(glu_clamp8_kernel, dim3(T, (F / 8 + 255) / 256), dim3(256), 0, (hipStream_t)stream, (const bf16*)sp, F,
                       limit, slope, (bf16*)out);
    return (int)hipGetLastError();
  }
  RowSrc s{sp, src_f32, slab, S};
  const long total = (long)T * F;
  hipLaunchKernelGGL(glu_clamp_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, s, F,
                     total, limit, slope, out, out_f32);
  return (int)hipGetLastError();
}

extern "C" int la_side_gate(const void* sp, int src_f32, long slab, int S, int T, int n, const void* tok,
                            const void* table, int ldt, int col0, void* out, int out_f32, void* stream) {
  using namespace la;
  if (T <= 0 || n <= 0 || !sp || !out || !tok || !table || col0 < 0 || col0 + n > ldt) return -1;
  RowSrc s{sp, src_f32, slab, S};
  const long total = (long)T * n;
  hipLaunchKernelGGL(side_gate_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, s, n,
                     total, (const int*)tok, (const bf16*)table, ldt, col0, out, out_f32);
  return (int)hipGetLastError();
}
