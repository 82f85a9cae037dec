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

// One wave per (token, chunk of head units); units are the H q heads, the G k heads and, when the
// values have columns of their own, G value heads that are only copied into the V page. A lane owns
// the rotary pairs p = lane, lane + 64, ... (elements p and p + rot_dims / 2 of the head) and the
// unrotated tail elements rot_dims + lane, ...: both elements of a pair live in one lane, so the
// rotation needs no exchange between lanes and no LDS, and the statistics of the head norm are one
// wave reduction. cos / sin of the lane's pairs are computed once per wave and kept in registers.
// K [blocks, G, 64, dk], V [blocks, G, 64, dv].
template <typename T>
__global__ void __launch_bounds__(256) rope_headnorm_cache_kernel(const RopeHeadnormParams P, int64_t T_rows, int hpw) {
  constexpr int MP = MAX_PAIRS / 64;        // pairs a lane can own
  constexpr int MT = MAX_HEAD / 64;         // tail elements a lane can own
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= T_rows) return;
  const int units = P.H + P.G + (P.v_off >= 0 ? P.G : 0);
  const int u0 = blockIdx.y * hpw, u1 = min(units, u0 + hpw);
  T* pr = (T*)P.proj + row * P.stride;
  const int p = P.pos[row] < 0 ? 0 : P.pos[row];
  const int half = P.rot_dims >> 1, dk = P.dk, tail = dk - P.rot_dims;
  float cs[MP], sn[MP];
#pragma unroll
  for (int j = 0; j < MP; ++j) {
    const int i = lane + 64 * j;
    cs[j] = 1.f;
    sn[j] = 0.f;
    if (i < half && u0 < P.H + P.G) {
      const double turns = (double)p * P.freq[i] * 0.15915494309189535;   // angle / 2 pi
      const float a = (float)((turns - floor(turns)) * 6.283185307179586);
      float s, c;
      sincosf(a, &s, &c);
      cs[j] = c * P.mag;
      sn[j] = s * P.mag;
    }
  }
  const int slot = P.slots[row];
  const int64_t page = slot >= 0 ? slot >> 6 : 0;
  const int in_page = slot & 63;
  for (int hh = u0; hh < u1; ++hh) {
    if (hh >= P.H + P.G) {   // a value head with columns of its own: page write only
      if (slot < 0) continue;
      const int g = hh - P.H - P.G;
      const T* vs = pr + P.v_off + (int64_t)g * P.dv;
      T* vd = (T*)P.vc + ((page * P.G + g) * 64 + in_page) * (int64_t)P.dv;
      for (int e = lane; e < P.dv; e += 64) vd[e] = vs[e];
      continue;
    }
    const bool is_k = hh >= P.H;
    const int g = hh - P.H;
    T* src = pr + (int64_t)hh * dk;
    const float* w = is_k ? P.k_w : P.q_w;
    float xa[MP], xb[MP], xt[MT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MP; ++j) {
      const int i = lane + 64 * j;
      xa[j] = i < half ? ldf(src + i) : 0.f;
      xb[j] = i < half ? ldf(src + half + i) : 0.f;
      ss += xa[j] * xa[j] + xb[j] * xb[j];
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int i = lane + 64 * j;
      xt[j] = i < tail ? ldf(src + P.rot_dims + i) : 0.f;
      ss += xt[j] * xt[j];
    }
    if (is_k && P.v_off < 0 && slot >= 0) {   // values = the keys as projected
      T* vd = (T*)P.vc + ((page * P.G + g) * 64 + in_page) * (int64_t)P.dv;
#pragma unroll
      for (int j = 0; j < MP; ++j) {
        const int i = lane + 64 * j;
        if (i < half) {
          stf(vd + i, xa[j]);
          stf(vd + half + i, xb[j]);
        }
      }
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        const int i = lane + 64 * j;
        if (i < tail) stf(vd + P.rot_dims + i, xt[j]);
      }
    }
    float r = 1.f;
    if (w != nullptr) {
      ss = wave_sum(ss);
      r = 1.0f / sqrtf(ss / (float)dk + P.eps);
    }
    T* kdst = (is_k && slot >= 0) ? (T*)P.kc + ((page * P.G + g) * 64 + in_page) * (int64_t)dk : nullptr;
#pragma unroll
    for (int j = 0; j < MP; ++j) {
      const int i = lane + 64 * j;
      if (i < half) {
        float u = xa[j], v = xb[j];
        if (w != nullptr) {
          u = u * r * w[i];
          v = v * r * w[half + i];
        }
        // (u, v) -> (u cos - v sin, v cos + u sin)
        const float ru = u * cs[j] - v * sn[j], rv = v * cs[j] + u * sn[j];
        stf(src + i, ru);
        stf(src + half + i, rv);
        if (kdst) {
          stf(kdst + i, ru);
          stf(kdst + half + i, rv);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int i = lane + 64 * j;
      if (i < tail) {
        const float v = w != nullptr ? xt[j] * r * w[P.rot_dims + i] : xt[j];
        if (w != nullptr) stf(src + P.rot_dims + i, v);
        if (kdst) stf(kdst + P.rot_dims + i, v);
      }
    }
  }
}

// bf16 rows, the rotation over the whole head (rot_dims = dk, dk % 16 == 0, dk / 2 a power of two
// up to 512), 16-byte aligned rows, columns and pages: a lane owns 8 neighbouring pairs - elements
// 8c .. 8c + 7 and the 8 elements half a head further - so every access is 16 bytes, a head takes
// CPH = dk / 16 lanes and a wave works on 64 / CPH heads at a time. cos / sin of the token go
// through the wave's LDS row (one sincos per lane). A wave takes the head rounds r = blockIdx.y,
// + gridDim.y, ...; the last y also copies value columns of their own into the V page.
__global__ void __launch_bounds__(256) rope_headnorm_cache_bf16x8_kernel(const RopeHeadnormParams P, int64_t T_rows) {
  __shared__ __attribute__((aligned(16))) float cs_all[4][MAX_PAIRS], sn_all[4][MAX_PAIRS];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= T_rows) return;
  float* cs = cs_all[wave];
  float* sn = sn_all[wave];
  uint16_t* pr = (uint16_t*)P.proj + row * P.stride;
  const int p = P.pos[row] < 0 ? 0 : P.pos[row];
  const int dk = P.dk, half = dk >> 1;
  for (int i = lane; i < half; i += 64) {
    const double turns = (double)p * P.freq[i] * 0.15915494309189535;   // angle / 2 pi
    const float a = (float)((turns - floor(turns)) * 6.283185307179586);
    float s, c;
    sincosf(a, &s, &c);
    cs[i] = c * P.mag;
    sn[i] = s * P.mag;
  }
  __builtin_amdgcn_wave_barrier();   // the wave's cos / sin rows are written (LDS ops of a wave complete in order)
  const int slot = P.slots[row];
  const int64_t page = slot >= 0 ? slot >> 6 : 0;
  const int in_page = slot & 63;
  const int CPH = half >> 3;               // lanes per head (a power of two <= 64)
  const int hpr = 64 / CPH;                // heads per round
  const int c8 = (lane & (CPH - 1)) * 8, hsub = lane / CPH;
  const int heads = P.H + P.G;
  float cc[8], sv[8];
#pragma unroll
  for (int j = 0; j < 8; j += 4) {
    const float4 c4 = *reinterpret_cast<const float4*>(cs + c8 + j), s4 = *reinterpret_cast<const float4*>(sn + c8 + j);
    cc[j] = c4.x, cc[j + 1] = c4.y, cc[j + 2] = c4.z, cc[j + 3] = c4.w;
    sv[j] = s4.x, sv[j + 1] = s4.y, sv[j + 2] = s4.z, sv[j + 3] = s4.w;
  }
  for (int h0 = blockIdx.y * hpr; h0 < heads; h0 += gridDim.y * hpr) {
    const int hh = h0 + hsub;
    const bool live = hh < heads;
    const bool is_k = hh >= P.H;
    const int g = hh - P.H;
    uint16_t* src = pr + (int64_t)(live ? hh : 0) * dk;
    const u16x8 ra = load8(src + c8), rb = load8(src + half + c8);
    if (live && is_k && P.v_off < 0 && slot >= 0) {   // values = the keys as projected
      uint16_t* vd = (uint16_t*)P.vc + ((page * P.G + g) * 64 + in_page) * (int64_t)P.dv;
      store8(vd + c8, ra);
      store8(vd + half + c8, rb);
    }
    float xa[8], xb[8], ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      xa[j] = bf2f(ra[j]);
      xb[j] = bf2f(rb[j]);
      ss += xa[j] * xa[j] + xb[j] * xb[j];
    }
    const float* w = is_k ? P.k_w : P.q_w;
    if (P.q_w != nullptr || P.k_w != nullptr) {   // (wave-uniform: the shuffles run in every lane)
      for (int o = CPH >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      if (live && w != nullptr) {
        const float r = 1.0f / sqrtf(ss / (float)dk + P.eps);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          xa[j] *= r * w[c8 + j];
          xb[j] *= r * w[half + c8 + j];
        }
      }
    }
    if (!live) continue;
    u16x8 oa, ob;
#pragma unroll
    for (int j = 0; j < 8; ++j) {   // (u, v) -> (u cos - v sin, v cos + u sin)
      oa[j] = f2bf(xa[j] * cc[j] - xb[j] * sv[j]);
      ob[j] = f2bf(xb[j] * cc[j] + xa[j] * sv[j]);
    }
    store8(src + c8, oa);
    store8(src + half + c8, ob);
    if (is_k && slot >= 0) {
      uint16_t* kd = (uint16_t*)P.kc + ((page * P.G + g) * 64 + in_page) * (int64_t)dk;
      store8(kd + c8, oa);
      store8(kd + half + c8, ob);
    }
  }
  if (P.v_off >= 0 && slot >= 0 && blockIdx.y == gridDim.y - 1) {
    const uint16_t* vs = pr + P.v_off;
    const int dv8 = P.dv >> 3;
    for (int c = lane; c < P.G * dv8; c += 64) {
      const int g = c / dv8, e = (c - g * dv8) * 8;
      store8((uint16_t*)P.vc + ((page * P.G + g) * 64 + in_page) * (int64_t)P.dv + e, load8(vs + (int64_t)g * P.dv + e));
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
  const int half = p.dk / 2;
  auto al16 = [](const void* q) { return ((uintptr_t)q % 16) == 0; };
  if (!f32 && p.rot_dims == p.dk && p.dk % 16 == 0 && (half & (half - 1)) == 0 && half <= 512 && p.stride % 8 == 0 &&
      al16(p.proj) && al16(p.kc) && al16(p.vc) && p.dv % 8 == 0 && (p.v_off < 0 || p.v_off % 8 == 0)) {
    const int hpr = 64 / (half / 8);
    const int rounds = (p.H + p.G + hpr - 1) / hpr;
    int gy = (int)(8192 / (T > 0 ? T : 1));            // enough waves to fill the chip when the tokens are few
    gy = gy < 1 ? 1 : (gy > rounds ? rounds : gy);
    rope_headnorm_cache_bf16x8_kernel<<<dim3((unsigned)((T + 3) / 4), (unsigned)gy), 256, 0, stream>>>(p, T);
    return;
  }
  // heads per wave: all of a token's heads in one wave once the tokens alone give ~4 waves per SIMD,
  // fewer when there are few tokens (single-token steps), so that the launch still fills the chip
  const int units = p.H + p.G + (p.v_off >= 0 ? p.G : 0);
  int hpw = (int)((T * units + 4095) / 4096);
  hpw = hpw < 1 ? 1 : (hpw > units ? units : hpw);
  const dim3 grid((unsigned)((T + 3) / 4), (unsigned)((units + hpw - 1) / hpw));
  if (f32)
    rope_headnorm_cache_kernel<float><<<grid, 256, 0, stream>>>(p, T, hpw);
  else
    rope_headnorm_cache_kernel<uint16_t><<<grid, 256, 0, stream>>>(p, T, hpw);
}

}  // namespace nga
