// Projection-side kernel of latent attention with a rotated key part (one workgroup per token):
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
#include "common.h"
#include "kernels.h"

namespace nga {

namespace {

constexpr int BS = 64;          // tokens per page
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

template <typename T>
__global__ void __launch_bounds__(256) latent_rope_cache_kernel(const LatentRopeParams P) {
  __shared__ float cs[MAX_PAIRS], sn[MAX_PAIRS];
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  T* pr = (T*)P.proj + row * P.stride;
  const int p = P.pos[row] < 0 ? 0 : P.pos[row];
  for (int i = tid; i < P.rot_dims / 2; i += blockDim.x) {
    const double turns = (double)p * P.freq[i] * 0.15915494309189535;   // angle / 2 pi
    const float a = (float)((turns - floor(turns)) * 6.283185307179586);
    float s, c;
    sincosf(a, &s, &c);
    cs[i] = c * P.mag;
    sn[i] = s * P.mag;
  }
  if (P.n_off >= 0) {
    float ss = 0.f;
    for (int c = tid; c < P.n_n; c += blockDim.x) {
      const float v = ldf(pr + P.n_off + c);
      ss += v * v;
    }
    ss = block_sum(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)P.n_n + P.eps);
    for (int c = tid; c < P.n_n; c += blockDim.x) stf(pr + P.n_off + c, ldf(pr + P.n_off + c) * r * P.n_w[c]);
  }
  __syncthreads();
  if (P.kv_off >= 0) {
    float ss = 0.f;
    for (int c = tid; c < P.r; c += blockDim.x) {
      const float v = ldf(pr + P.kv_off + c);
      ss += v * v;
    }
    ss = block_sum(ss, red);
    const int slot = P.slots[row];
    if (slot >= 0) {
      const float r = 1.0f / sqrtf(ss / (float)P.r + P.eps);
      T* dst = (T*)P.page + ((int64_t)(slot / BS) * BS + slot % BS) * (P.r + P.rot_dim);
      for (int c = tid; c < P.r; c += blockDim.x) stf(dst + c, ldf(pr + P.kv_off + c) * r * P.kv_w[c]);
      const T* kr = pr + P.kv_off + P.r;
      for (int e = tid; e < P.rot_dim; e += blockDim.x)
        stf(dst + P.r + e, rotated(kr, e, P.rot_dims, P.interleaved != 0, cs, sn));
    }
  }
  if (P.q_off >= 0) {
    const int qd = P.dim + P.rot_dim;
    T* qo = (T*)P.q_out + row * P.q_out_stride;
    for (int i = tid; i < P.heads * P.rot_dim; i += blockDim.x) {
      const int h = i / P.rot_dim, e = i - h * P.rot_dim;
      stf(qo + (int64_t)h * P.q_w + (P.q_w - P.rot_dim) + e,
          rotated(pr + P.q_off + (int64_t)h * qd + P.dim, e, P.rot_dims, P.interleaved != 0, cs, sn));
    }
  }
}

}  // namespace

void launch_latent_rope_cache(const LatentRopeParams& p, int64_t T, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (p.rot_dims / 2 > MAX_PAIRS) abort();   // the binding checks rot_dims <= 512
  if (f32)
    latent_rope_cache_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>(p);
  else
    latent_rope_cache_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>(p);
}

}  // namespace nga
