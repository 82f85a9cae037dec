// Projection-side kernels that apply rotary positions from a frequency table (one wave per token).
//
// latent_rope_cache: latent attention with a rotated key part:
//
//   * optional RMS norm, in place, of a column range (a query latent in front of its
//     up-projection);
//   * the latent [r] RMS-normalised and the rotated key part [rot_dim] that all heads share, with
//     rotary positions, written into the token's page slot: page row = [latent | rotated part];
//   * rotary positions on the rotated part of every query head, written behind the columns that
//     the folded unrotated query takes in the attention's query rows.
//
// Rotary positions act on the first rot_dims elements of a rotated part. Pair i turns by
// pos * freq[i]: the product is taken in float64 and reduced to one turn before the fp32 sincos,
// so the angle is exact to fp32 at any position. Pairs are (2i, 2i + 1) (interleaved) or
// (i, i + rot_dims / 2). cos and sin carry a common factor (frequency-scaled rotations).
// Norm statistics, rotations and sums are fp32 whatever the activation type.
//
// rope_headnorm_cache: GQA attention rows [q heads | k heads | ...]: optional RMS norm of every q
// and k head (one weight vector each), rotary positions on the first rot_dims elements of every
// head (pairs (i, i + rot_dims / 2)), q and k written back, K and V page write; the values are
// columns of the row or the k heads as they were before norm and rotation.
#include "common.h"
#include "kernels.h"

namespace nga {

namespace {

constexpr int MAX_PAIRS = 256;  // rot_dims <= 512

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// element e of a rotated part after the rotation (src: the part's first element)
template <typename T>
__device__ __forceinline__ float rotated(const T* src, int e, int n, bool interleaved, const float* cs,
                                         const float* sn) {
  if (e >= n) return ldf(src + e);
  int pair, other;
  bool first;
  if (interleaved) {
    pair = e >> 1;
    first = (e & 1) == 0;
    other = e ^ 1;
  } else {
    const int half = n >> 1;
    first = e < half;
    pair = first ? e : e - half;
    other = first ? e + half : e - half;
  }
  const float a = ldf(src + e), b = ldf(src + other);
  // (u, v) -> (u cos - v sin, v cos + u sin)
  return first ? a * cs[pair] - b * sn[pair] : a * cs[pair] + b * sn[pair];
}

// One wave per token, four tokens per workgroup: the norm statistics are wave reductions and the
// cos / sin of the token live in the wave's own LDS rows, so no workgroup barrier is needed.
template <typename T>
__global__ void __launch_bounds__(256) latent_rope_cache_kernel(const LatentRopeParams P, int64_t T_rows) {
  __shared__ float cs_all[4][MAX_PAIRS], sn_all[4][MAX_PAIRS];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= T_rows) return;
  float* cs = cs_all[wave];
  float* sn = sn_all[wave];
  T* pr = (T*)P.proj + row * P.stride;
  const int p = P.pos[row] < 0 ? 0 : P.pos[row];
  for (int i = lane; i < P.rot_dims / 2; i += 64) {
    const double turns = (double)p * P.freq[i] * 0.15915494309189535;   // angle / 2 pi
    const float a = (float)((turns - floor(turns)) * 6.283185307179586);
    float s, c;
    sincosf(a, &s, &c);
    cs[i] = c * P.mag;
    sn[i] = s * P.mag;
  }
  if (P.n_off >= 0) {
    float ss = 0.f;
    for (int c = lane; c < P.n_n; c += 64) {
      const float v = ldf(pr + P.n_off + c);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)P.n_n + P.eps);
    for (int c = lane; c < P.n_n; c += 64) stf(pr + P.n_off + c, ldf(pr + P.n_off + c) * r * P.n_w[c]);
  }
  __builtin_amdgcn_wave_barrier();   // the wave's cos / sin rows are written (LDS ops of a wave complete in order)
  if (P.kv_off >= 0) {
    const int slot = P.slots[row];
    if (slot >= 0) {
      float ss = 0.f;
      for (int c = lane; c < P.r; c += 64) {
        const float v = ldf(pr + P.kv_off + c);
        ss += v * v;
      }
      ss = wave_sum(ss);
      const float r = 1.0f / sqrtf(ss / (float)P.r + P.eps);
      T* dst = (T*)P.page + (int64_t)slot * (P.r + P.rot_dim);   // page rows are contiguous: slot = page * 64 + offset
      for (int c = lane; c < P.r; c += 64) stf(dst + c, ldf(pr + P.kv_off + c) * r * P.kv_w[c]);
      const T* kr = pr + P.kv_off + P.r;
      for (int e = lane; e < P.rot_dim; e += 64)
        stf(dst + P.r + e, rotated(kr, e, P.rot_dims, P.interleaved != 0, cs, sn));
    }
  }
  if (P.q_off >= 0) {
    // element e of every head's rotated part: the pair, its partner and cos / sin are the lane's
    // own for all heads
    const int qd = P.dim + P.rot_dim;
    T* qo = (T*)P.q_out + row * P.q_out_stride + (P.q_w - P.rot_dim);
    const T* qi = pr + P.q_off + P.dim;
    for (int e = lane; e < P.rot_dim; e += 64) {
      if (e >= P.rot_dims) {
        for (int h = 0; h < P.heads; ++h) stf(qo + (int64_t)h * P.q_w + e, ldf(qi + (int64_t)h * qd + e));
        continue;
      }
      int pair, other;
      bool first;
      if (P.interleaved) {
        pair = e >> 1;
        first = (e & 1) == 0;
        other = e ^ 1;
      } else {
        const int half = P.rot_dims >> 1;
        first = e < half;
        pair = first ? e : e - half;
        other = first ? e + half : e - half;
      }
      const float c = cs[pair], s = first ? -sn[pair] : sn[pair];
      for (int h = 0; h < P.heads; ++h) {
        const T* src = qi + (int64_t)h * qd;
        stf(qo + (int64_t)h * P.q_w + e, ldf(src + e) * c + ldf(src + other) * s);
      }
    }
  }
}

constexpr int MAX_HEAD = 512;   // widest q / k head of rope_headnorm_cache

// One wave per token, four tokens per workgroup. A head goes through the wave's LDS row: raw
// values in, statistics by wave reduction, normalised values back into the row, then every lane
// reads its element and the element's rotation partner. K [blocks, G, 64, dk], V [blocks, G, 64, dv].
template <typename T>
__global__ void __launch_bounds__(256) rope_headnorm_cache_kernel(const RopeHeadnormParams P, int64_t T_rows) {
  __shared__ float cs_all[4][MAX_PAIRS], sn_all[4][MAX_PAIRS];
  __shared__ float hd_all[4][MAX_HEAD];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= T_rows) return;
  float* cs = cs_all[wave];
  float* sn = sn_all[wave];
  float* hd = hd_all[wave];
  T* pr = (T*)P.proj + row * P.stride;
  const int p = P.pos[row] < 0 ? 0 : P.pos[row];
  const int half = P.rot_dims >> 1;
  for (int i = lane; i < half; i += 64) {
    const double turns = (double)p * P.freq[i] * 0.15915494309189535;   // angle / 2 pi
    const float a = (float)((turns - floor(turns)) * 6.283185307179586);
    float s, c;
    sincosf(a, &s, &c);
    cs[i] = c * P.mag;
    sn[i] = s * P.mag;
  }
  const int slot = P.slots[row];
  const int64_t page = slot >= 0 ? slot >> 6 : 0;
  const int in_page = slot & 63;
  const int dk = P.dk;
  for (int hh = 0; hh < P.H + P.G; ++hh) {
    const bool is_k = hh >= P.H;
    const int g = hh - P.H;
    T* src = pr + (int64_t)hh * dk;
    const float* w = is_k ? P.k_w : P.q_w;
    float ss = 0.f;
    for (int e = lane; e < dk; e += 64) {
      const float v = ldf(src + e);
      hd[e] = v;
      ss += v * v;
      if (is_k && P.v_off < 0 && slot >= 0)     // values = the keys as projected
        stf((T*)P.vc + ((page * P.G + g) * 64 + in_page) * (int64_t)P.dv + e, v);
    }
    if (w != nullptr) {
      ss = wave_sum(ss);
      const float r = 1.0f / sqrtf(ss / (float)dk + P.eps);
      for (int e = lane; e < dk; e += 64) hd[e] = hd[e] * r * w[e];   // a lane rewrites its own elements
    }
    __builtin_amdgcn_wave_barrier();   // the wave's LDS rows are written (LDS ops of a wave complete in order)
    T* kdst = (is_k && slot >= 0) ? (T*)P.kc + ((page * P.G + g) * 64 + in_page) * (int64_t)dk : nullptr;
    for (int e = lane; e < dk; e += 64) {
      float v = hd[e];
      if (e < P.rot_dims) {
        const bool first = e < half;
        const int pair = first ? e : e - half;
        const float o = hd[first ? e + half : e - half];
        // (u, v) -> (u cos - v sin, v cos + u sin)
        v = first ? v * cs[pair] - o * sn[pair] : v * cs[pair] + o * sn[pair];
      }
      stf(src + e, v);
      if (kdst) stf(kdst + e, v);
    }
    __builtin_amdgcn_wave_barrier();   // every lane has read the row before the next head overwrites it
  }
  if (P.v_off >= 0 && slot >= 0) {
    const T* vs = pr + P.v_off;
    for (int c = lane; c < P.G * P.dv; c += 64) {
      const int g = c / P.dv, e = c - g * P.dv;
      stf((T*)P.vc + ((page * P.G + g) * 64 + in_page) * (int64_t)P.dv + e, ldf(vs + c));
    }
  }
}

}  // namespace

void launch_latent_rope_cache(const LatentRopeParams& p, int64_t T, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (p.rot_dims / 2 > MAX_PAIRS) abort();   // the binding checks rot_dims <= 512
  const dim3 grid((unsigned)((T + 3) / 4));
  if (f32)
    latent_rope_cache_kernel<float><<<grid, 256, 0, stream>>>(p, T);
  else
    latent_rope_cache_kernel<uint16_t><<<grid, 256, 0, stream>>>(p, T);
}

void launch_rope_headnorm_cache(const RopeHeadnormParams& p, int64_t T, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (p.rot_dims / 2 > MAX_PAIRS || p.dk > MAX_HEAD) abort();   // the binding checks both
  const dim3 grid((unsigned)((T + 3) / 4));
  if (f32)
    rope_headnorm_cache_kernel<float><<<grid, 256, 0, stream>>>(p, T);
  else
    rope_headnorm_cache_kernel<uint16_t><<<grid, 256, 0, stream>>>(p, T);
}

}  // namespace nga
