// Rotary positions on projection rows and the append of keys / values into the paged pools, for
// designs whose key and value widths differ, whose rotation covers part of a head at an offset, and
// whose frequencies are a table (YaRN-scaled or plain) rather than one base.
//
//   rope_pages:  row [q (H x Dq) | k (G x Dk) | v (G x Dv)];  dims [q_off, q_off + rot) of every
//                query head and [0, rot) of every key head are rotated, pair (2i, 2i + 1)
//                (interleaved) or (i, i + rot / 2):  (u, v) -> (u c - v s, v c + u s), angle
//                pos * freq[i] formed and evaluated in fp32, c and s times `mag`.
//                K rows go to [blocks][G][BS][Dk], V to [blocks][G][BS / 8][Dv][8].
//   latent_kv:   row [c (rank) | r (rot)]:  c / sqrt(mean c^2 + eps) * w and the rotated r are stored
//                as ONE row of a one-head K pool, [blocks][1][BS][rank + rot]: key and value at once.
//
//   qk_norm_pages: no rotation: every query and key head divided by its root mean square (fp32,
//                no weight), queries times a temperature 1 + coef ln(floor((pos + 1) / every) + 1);
//                K / V appended as above.  A wave per head.
//   sinusoid_add: additive positions on the fp32 stream, column 2i += sin(pos f_i), 2i + 1 += cos.
//
// A workgroup per token; the token's cos / sin are computed once into LDS.
#include "common.h"

namespace la {

constexpr int RP_NT = 256;

// rotated value of dim d (relative to the start of the rotated span) of a head whose span starts at x
template <typename AT>
LA_DEV float rot_dim(const AT* __restrict__ x, int d, int rot, int interleaved, const float* __restrict__ cs) {
  const int half = rot >> 1;
  int i, first;
  float u, v;
  if (interleaved) {
    i = d >> 1;
    first = !(d & 1);
    u = (float)x[d & ~1];
    v = (float)x[d | 1];
  } else {
    first = d < half;
    i = first ? d : d - half;
    u = (float)x[i];
    v = (float)x[i + half];
  }
  const float c = cs[2 * i], s = cs[2 * i + 1];
  return first ? u * c - v * s : v * c + u * s;
}

LA_DEV void fill_cos_sin(float* cs, int rot, int p, const float* __restrict__ freqs, float mag) {
  for (int i = threadIdx.x; i < (rot >> 1); i += blockDim.x) {
    const float a = (float)p * freqs[i];
    cs[2 * i] = cosf(a) * mag;
    cs[2 * i + 1] = sinf(a) * mag;
  }
}

template <typename AT>
__global__ __launch_bounds__(RP_NT) void rope_pages_kernel(const AT* __restrict__ src, int H, int Dq, int G, int Dk, int Dv,
                                                           const int* __restrict__ pos, const int* __restrict__ slots,
                                                           const float* __restrict__ freqs, float mag, int rot, int q_off,
                                                           int interleaved, AT* __restrict__ q_out, AT* __restrict__ kc,
                                                           AT* __restrict__ vc, int BS) {
  extern __shared__ float cs[];          // [rot / 2][2]
  const int t = blockIdx.x, tid = threadIdx.x;
  const int Cq = H * Dq, Ck = G * Dk, Cv = G * Dv;
  const AT* row = src + (long)t * (Cq + Ck + Cv);
  fill_cos_sin(cs, rot, pos[t], freqs, mag);
  __syncthreads();
  for (int e = tid; e < Cq; e += RP_NT) {
    const int h = e / Dq, d = e - h * Dq;
    float o;
    if (d >= q_off && d < q_off + rot) o = rot_dim<AT>(row + h * Dq + q_off, d - q_off, rot, interleaved, cs);
    else o = (float)row[e];
    q_out[(long)t * Cq + e] = (AT)o;
  }
  if (!G) return;
  const int slot = slots[t];
  if (slot < 0) return;
  const int blk = slot / BS, off = slot - blk * BS;
  for (int e = tid; e < Ck; e += RP_NT) {
    const int g = e / Dk, d = e - g * Dk;
    const float o = d < rot ? rot_dim<AT>(row + Cq + g * Dk, d, rot, interleaved, cs) : (float)row[Cq + e];
    kc[(((long)blk * G + g) * BS + off) * Dk + d] = (AT)o;
  }
  for (int e = tid; e < Cv; e += RP_NT) {
    const int g = e / Dv, d = e - g * Dv;
    vc[((((long)blk * G + g) * (BS >> 3) + (off >> 3)) * Dv + d) * 8 + (off & 7)] = row[Cq + Ck + e];
  }
}

template <typename AT>
__global__ __launch_bounds__(RP_NT) void latent_kv_kernel(const AT* __restrict__ src, int rank, int rot,
                                                          const float* __restrict__ w, float eps,
                                                          const int* __restrict__ pos, const int* __restrict__ slots,
                                                          const float* __restrict__ freqs, float mag, int interleaved,
                                                          AT* __restrict__ kc, int BS) {
  extern __shared__ float cs[];          // [rot / 2][2]
  __shared__ float red[RP_NT / 64];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int slot = slots[t];
  if (slot < 0) return;                  // uniform over the workgroup
  const int W = rank + rot;
  const AT* row = src + (long)t * W;
  fill_cos_sin(cs, rot, pos[t], freqs, mag);
  float ss = 0.f;
  for (int c = tid; c < rank; c += RP_NT) {
    const float x = (float)row[c];
    ss = fmaf(x, x, ss);
  }
  ss = block_sum<RP_NT>(ss, red);        // its barriers also publish cs
  const float inv = 1.f / sqrtf(ss / (float)rank + eps);
  AT* dst = kc + (long)slot * W;         // one head: page row = slot
  for (int c = tid; c < rank; c += RP_NT) dst[c] = (AT)((float)row[c] * inv * w[c]);
  for (int d = tid; d < rot; d += RP_NT) dst[rank + d] = (AT)rot_dim<AT>(row + rank, d, rot, interleaved, cs);
  (void)BS;
}

// row [q (H x Dq) | k (G x Dk) | v (G x Dv)] with row stride ld: unit-RMS q (times the position's
// temperature) -> q_out, unit-RMS k and v -> pages.  Wave w of the workgroup takes heads w, w + 4, ...
template <typename AT>
__global__ __launch_bounds__(RP_NT) void qk_norm_pages_kernel(const AT* __restrict__ src, long ld, int H, int Dq, int G,
                                                              int Dk, int Dv, const int* __restrict__ pos,
                                                              const int* __restrict__ slots, float eps, float coef,
                                                              int every, AT* __restrict__ q_out, AT* __restrict__ kc,
                                                              AT* __restrict__ vc, int BS) {
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int Cq = H * Dq, Ck = G * Dk, Cv = G * Dv;
  const AT* row = src + (long)t * ld;
  float tau = 1.f;
  if (every > 0) tau = 1.f + coef * logf((float)((pos[t] + 1) / every + 1));
  const int slot = G ? slots[t] : -1;
  const int blk = slot >= 0 ? slot / BS : 0, off = slot >= 0 ? slot - blk * BS : 0;
  for (int u = wave; u < H + G; u += RP_NT / 64) {
    const bool isq = u < H;
    if (!isq && slot < 0) continue;
    const int n = isq ? Dq : Dk;
    const AT* x = isq ? row + (long)u * Dq : row + Cq + (long)(u - H) * Dk;
    float ss = 0.f;
    for (int d = lane; d < n; d += 64) {
      const float v = (float)x[d];
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    const float f = (1.f / sqrtf(ss / (float)n + eps)) * (isq ? tau : 1.f);
    AT* dst = isq ? q_out + (long)t * Cq + (long)u * Dq : kc + (((long)blk * G + (u - H)) * BS + off) * Dk;
    for (int d = lane; d < n; d += 64) dst[d] = (AT)((float)x[d] * f);
  }
  if (slot < 0) return;
  for (int e = tid; e < Cv; e += RP_NT) {
    const int g = e / Dv, d = e - g * Dv;
    vc[((((long)blk * G + g) * (BS >> 3) + (off >> 3)) * Dv + d) * 8 + (off & 7)] = row[Cq + Ck + e];
  }
}

__global__ __launch_bounds__(256) void sinusoid_add_kernel(float* __restrict__ res, int D, const int* __restrict__ pos,
                                                           const float* __restrict__ freqs) {
  const int t = blockIdx.x;
  const float p = (float)pos[t];
  for (int i = threadIdx.x; 2 * i < D; i += 256) {
    const float a = p * freqs[i];
    float* r = res + (long)t * D + 2 * i;
    r[0] += sinf(a);
    if (2 * i + 1 < D) r[1] += cosf(a);
  }
}

// A workgroup per token: per-head RMS norm with a weight on q and k (a wave per head), rotation of their
// first `rot` dims in the (i, i + rot / 2) layout, values rotated over their whole width with their own
// frequency table (vfreqs null: values pass), q -> q_out, K / V -> pages.
template <typename AT>
__global__ __launch_bounds__(RP_NT) void qk_norm_rope_pages_kernel(
    const AT* __restrict__ src, long ld, int H, int D, int G, int Dv, const int* __restrict__ pos,
    const int* __restrict__ slots, const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const float* __restrict__ freqs, float mag, int rot, const float* __restrict__ vfreqs, AT* __restrict__ q_out,
    AT* __restrict__ kc, AT* __restrict__ vc, int BS) {
  extern __shared__ float cs[];          // [rot / 2][2] for q / k, then [Dv / 2][2] for v
  float* vcs = cs + rot;
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int Cq = H * D, Ck = G * D, Cv = G * Dv, half = rot >> 1, vhalf = Dv >> 1;
  const AT* row = src + (long)t * ld;
  const int p = pos[t];
  // both tables in one pass, a thread per angle, sine and cosine from one evaluation
  for (int i = tid; i < half + (vfreqs ? vhalf : 0); i += RP_NT) {
    const bool isv = i >= half;
    const int k = isv ? i - half : i;
    float sn, c;
    sincosf((float)p * (isv ? vfreqs[k] : freqs[k]), &sn, &c);
    float* dst = isv ? vcs : cs;
    const float m = isv ? 1.f : mag;
    dst[2 * k] = c * m;
    dst[2 * k + 1] = sn * m;
  }
  __syncthreads();
  const int slot = slots[t];
  const int blk = slot >= 0 ? slot / BS : 0, off = slot >= 0 ? slot - blk * BS : 0;
  for (int u = wave; u < H + G; u += RP_NT / 64) {
    const bool isq = u < H;
    if (!isq && slot < 0) continue;
    const AT* x = isq ? row + (long)u * D : row + Cq + (long)(u - H) * D;
    const float* w = isq ? qw : kw;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float v = (float)x[d];
      ss = fmaf(v, v, ss);
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
    AT* dst = isq ? q_out + (long)t * Cq + (long)u * D : kc + (((long)blk * G + (u - H)) * BS + off) * D;
    for (int d = lane; d < D; d += 64) {
      float y;
      if (d < rot) {
        const bool first = d < half;
        const int i = first ? d : d - half;
        const float a = (float)x[i] * inv * w[i], b = (float)x[i + half] * inv * w[i + half];
        const float c = cs[2 * i], sn = cs[2 * i + 1];
        y = first ? a * c - b * sn : b * c + a * sn;
      } else {
        y = (float)x[d] * inv * w[d];
      }
      dst[d] = (AT)y;
    }
  }
  if (slot < 0) return;
  for (int e = tid; e < Cv; e += RP_NT) {
    const int g = e / Dv, d = e - g * Dv;
    const AT* x = row + Cq + Ck + (long)g * Dv;
    AT y = x[d];
    if (vfreqs) {
      const bool first = d < vhalf;
      const int i = first ? d : d - vhalf;
      const float a = (float)x[i], b = (float)x[i + vhalf], c = vcs[2 * i], sn = vcs[2 * i + 1];
      y = (AT)(first ? a * c - b * sn : b * c + a * sn);
    }
    vc[((((long)blk * G + g) * (BS >> 3) + (off >> 3)) * Dv + d) * 8 + (off & 7)] = y;
  }
}

// every head of a row turned over its whole width, dims m and m + Dv / 2 by sign * pos * freqs[m], times scale
template <typename AT>
__global__ __launch_bounds__(RP_NT) void rotate_heads_kernel(const AT* __restrict__ x, int H, int Dv,
                                                             const int* __restrict__ pos, const float* __restrict__ freqs,
                                                             float sign, float scale, AT* __restrict__ out, long ldo) {
  extern __shared__ float cs[];          // [Dv / 2][2]
  const int t = blockIdx.x, vhalf = Dv >> 1;
  for (int i = threadIdx.x; i < vhalf; i += RP_NT) {
    float sn, c;
    sincosf(sign * ((float)pos[t] * freqs[i]), &sn, &c);
    cs[2 * i] = c * scale;
    cs[2 * i + 1] = sn * scale;
  }
  __syncthreads();
  const AT* row = x + (long)t * H * Dv;
  for (int e = threadIdx.x; e < H * vhalf; e += RP_NT) {
    const int h = e / vhalf, i = e - h * vhalf;
    const float a = (float)row[h * Dv + i], b = (float)row[h * Dv + i + vhalf], c = cs[2 * i], sn = cs[2 * i + 1];
    out[(long)t * ldo + h * Dv + i] = (AT)(a * c - b * sn);
    out[(long)t * ldo + h * Dv + i + vhalf] = (AT)(b * c + a * sn);
  }
}

}  // namespace la

extern "C" int la_qk_norm_rope_pages(int f32, const void* src, long ld, int T, int H, int D, int G, int Dv, const void* pos,
                                     const void* slots, const void* qw, const void* kw, float eps, const void* freqs,
                                     float mag, int rot, const void* vfreqs, void* q_out, void* kc, void* vc, int BS,
                                     void* stream) {
  using namespace la;
  if (T <= 0 || H <= 0 || D <= 0 || G <= 0 || Dv <= 0 || (rot & 1) || rot < 0 || rot > D || (vfreqs && (Dv & 1))) return -1;
  if (ld < (long)(H + G) * D + (long)G * Dv || BS <= 0 || (BS & 7)) return -2;
  if (!src || !pos || !slots || !qw || !kw || (rot > 0 && !freqs) || !q_out || !kc || !vc) return -3;
  const size_t shm = (size_t)(rot + Dv + 2) * sizeof(float);
  if (f32)
    hipLaunchKernelGGL(qk_norm_rope_pages_kernel<float>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const float*)src,
                       ld, H, D, G, Dv, (const int*)pos, (const int*)slots, (const float*)qw, (const float*)kw, eps,
                       (const float*)freqs, mag, rot, (const float*)vfreqs, (float*)q_out, (float*)kc, (float*)vc, BS);
  else
    hipLaunchKernelGGL(qk_norm_rope_pages_kernel<bf16>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const bf16*)src, ld,
                       H, D, G, Dv, (const int*)pos, (const int*)slots, (const float*)qw, (const float*)kw, eps,
                       (const float*)freqs, mag, rot, (const float*)vfreqs, (bf16*)q_out, (bf16*)kc, (bf16*)vc, BS);
  return (int)hipGetLastError();
}

extern "C" int la_rotate_heads(int f32, const void* x, int T, int H, int Dv, const void* pos, const void* freqs, float sign,
                               float scale, void* out, long ldo, void* stream) {
  using namespace la;
  if (T <= 0 || H <= 0 || Dv <= 0 || (Dv & 1) || ldo < (long)H * Dv || !x || !pos || !freqs || !out) return -1;
  const size_t shm = (size_t)(Dv + 2) * sizeof(float);
  if (f32)
    hipLaunchKernelGGL(rotate_heads_kernel<float>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const float*)x, H, Dv,
                       (const int*)pos, (const float*)freqs, sign, scale, (float*)out, ldo);
  else
    hipLaunchKernelGGL(rotate_heads_kernel<bf16>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const bf16*)x, H, Dv,
                       (const int*)pos, (const float*)freqs, sign, scale, (bf16*)out, ldo);
  return (int)hipGetLastError();
}

extern "C" int la_qk_norm_pages(int f32, const void* src, int ld, int T, int H, int Dq, int G, int Dk, int Dv,
                                const void* pos, const void* slots, float eps, float coef, int every, void* q_out,
                                void* kc, void* vc, int BS, void* stream) {
  using namespace la;
  if (T <= 0 || H <= 0 || Dq <= 0 || G < 0 || every < 0 || ld < H * Dq + G * Dk + G * Dv) return -1;
  if (G && (Dk <= 0 || Dv <= 0 || !kc || !vc || !slots || BS <= 0 || (BS & 7))) return -2;
  if (!src || !pos || !q_out) return -3;
  if (f32)
    hipLaunchKernelGGL(qk_norm_pages_kernel<float>, dim3(T), dim3(RP_NT), 0, (hipStream_t)stream, (const float*)src, (long)ld,
                       H, Dq, G, Dk, Dv, (const int*)pos, (const int*)slots, eps, coef, every, (float*)q_out, (float*)kc,
                       (float*)vc, BS);
  else
    hipLaunchKernelGGL(qk_norm_pages_kernel<bf16>, dim3(T), dim3(RP_NT), 0, (hipStream_t)stream, (const bf16*)src, (long)ld,
                       H, Dq, G, Dk, Dv, (const int*)pos, (const int*)slots, eps, coef, every, (bf16*)q_out, (bf16*)kc,
                       (bf16*)vc, BS);
  return (int)hipGetLastError();
}

extern "C" int la_sinusoid_add(void* res, int T, int D, const void* pos, const void* freqs, void* stream) {
  using namespace la;
  if (T <= 0 || D <= 0 || !res || !pos || !freqs) return -1;
  hipLaunchKernelGGL(sinusoid_add_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, (float*)res, D, (const int*)pos,
                     (const float*)freqs);
  return (int)hipGetLastError();
}

extern "C" int la_rope_pages(int f32, const void* src, int T, int H, int Dq, int G, int Dk, int Dv, const void* pos,
                             const void* slots, const void* freqs, float mag, int rot, int q_off, int interleaved,
                             void* q_out, void* kc, void* vc, int BS, void* stream) {
  using namespace la;
  if (T <= 0 || H <= 0 || Dq <= 0 || G < 0 || (rot & 1) || rot < 0 || q_off < 0 || q_off + rot > Dq) return -1;
  if (G && (rot > Dk || !kc || !vc || !slots || BS <= 0 || (BS & 7))) return -2;
  if (!src || !pos || !freqs || !q_out) return -3;
  const size_t shm = (size_t)(rot > 0 ? rot : 2) * sizeof(float);
  if (f32)
    hipLaunchKernelGGL(rope_pages_kernel<float>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const float*)src, H, Dq,
                       G, Dk, Dv, (const int*)pos, (const int*)slots, (const float*)freqs, mag, rot, q_off, interleaved,
                       (float*)q_out, (float*)kc, (float*)vc, BS);
  else
    hipLaunchKernelGGL(rope_pages_kernel<bf16>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const bf16*)src, H, Dq, G,
                       Dk, Dv, (const int*)pos, (const int*)slots, (const float*)freqs, mag, rot, q_off, interleaved,
                       (bf16*)q_out, (bf16*)kc, (bf16*)vc, BS);
  return (int)hipGetLastError();
}

extern "C" int la_latent_kv(int f32, const void* src, int T, int rank, int rot, const void* w, float eps, const void* pos,
                            const void* slots, const void* freqs, float mag, int interleaved, void* kc, int BS,
                            void* stream) {
  using namespace la;
  if (T <= 0 || rank <= 0 || rot < 0 || (rot & 1) || !src || !w || !pos || !slots || !freqs || !kc) return -1;
  const size_t shm = (size_t)(rot > 0 ? rot : 2) * sizeof(float);
  if (f32)
    hipLaunchKernelGGL(latent_kv_kernel<float>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const float*)src, rank,
                       rot, (const float*)w, eps, (const int*)pos, (const int*)slots, (const float*)freqs, mag, interleaved,
                       (float*)kc, BS);
  else
    hipLaunchKernelGGL(latent_kv_kernel<bf16>, dim3(T), dim3(RP_NT), shm, (hipStream_t)stream, (const bf16*)src, rank, rot,
                       (const float*)w, eps, (const int*)pos, (const int*)slots,
                       (const float*)freqs, mag, interleaved, (bf16*)kc, BS);
  return (int)hipGetLastError();
}
