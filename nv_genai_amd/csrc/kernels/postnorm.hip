// Row kernels of post-norm decoders with an fp32 residual stream and a token-shift state:
//
//   embed_pos         x[t]  = embed[id[t]] + pos_table[pos[t]]                    (fp32 out)
//   rmsnorm_residual  x[t] += y[t] * rsqrt(mean(y[t]^2) + eps) * w  (+ a cast copy of x[t])
//   token_shift       h[t]  = x[t] + (prev(t) - x[t]) * mu, prev(t) the same layer's input one
//                     token earlier: a row of this step, a state slot, or zeros (position 0)
//   shift_save        state[slot[i]] = x[last_row[i]] for every sequence of the step
//   glu_gelu_tanh     [T, 2F] = [gate | up] -> gelu_tanh(gate) * up, any F, bf16 or fp32
//   embed_rows        x[t]  = embed[id[t]] * scale                                (fp32 out)
//   rmsnorm_residual_next   x[t] += rmsnorm(y[t]) * w, out[t] = rmsnorm(x[t]) * next_w: the
//                     post-norm of one sub-layer and the pre-norm of the next in one pass
//                     (weights of H elements or of one: a single gain)
//   relu_sq           relu(x)^2
//   softcap           z = cap * tanh(z * scale / cap) on fp32 logits
//   residual_add_rmsnorm   x[t] += y[t], out[t] = rmsnorm(x[t]) * w: the residual sum of one
//                     pre-norm sub-layer and the norm in front of the next in one pass
//   clamped_glu       [gate F | up F | ...] -> g sigmoid(alpha g) (u + shift), g = min(gate, limit),
//                     u = clamp(up, +-limit), optionally times sigmoid of one gate column of the row
//   group_rmsnorm     RMS norm of each of G equal column groups of fp32 rows (heads), weight per
//                     group element or per column, optional sigmoid gate per column
//   dyt_norm          tanh(alpha x) * w + b of fp32 rows (dynamic tanh in place of a norm)
//   residual_dyt      x += (y1 + y2 + bias), or x = y1, and the dynamic tanh of the result:
//                     the step between two parallel layers in one pass
//   pack_pair         [a | b] rows of two fp32 streams in the activation type
//   bias_gelu_tanh    gelu_tanh(x + bias) in place, fp32 bias, any width
//
// The residual, the norms and the shift interpolation are fp32 whatever the activation type T
// (bf16 storage as uint16_t, or float). Memory-bound: one workgroup per row, columns strided
// over the lanes (no alignment assumed: widths need not be multiples of 8).
#include "common.h"
#include "kernels.h"

namespace nga {

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

template <typename T>
__global__ void __launch_bounds__(256) embed_pos_kernel(float* __restrict__ x, const int32_t* __restrict__ ids,
                                                        const int32_t* __restrict__ pos, const T* __restrict__ embed,
                                                        const T* __restrict__ ptab, int H, int vocab, int max_pos) {
  const int64_t row = blockIdx.x;
  int id = ids[row], p = pos[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // padding rows of a captured step
  p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
  for (int c = threadIdx.x; c < H; c += blockDim.x)
    x[row * H + c] = ldf(embed + (int64_t)id * H + c) + ldf(ptab + (int64_t)p * H + c);
}

template <typename T>
__global__ void __launch_bounds__(256) rmsnorm_residual_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                               int64_t y_stride, const float* __restrict__ w,
                                                               float eps, int H, T* __restrict__ cast_out) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float v = ldf(yr + c);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float v = x[row * H + c] + ldf(yr + c) * r * w[c];
    x[row * H + c] = v;
    if (cast_out) stf(cast_out + row * H + c, v);
  }
}

// out = rmsnorm(x) * w of fp32 rows (the model's last norm), written in T
template <typename T>
__global__ void __launch_bounds__(256) rmsnorm_f32_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                          const int64_t* __restrict__ rows, const float* __restrict__ w,
                                                          float eps, int H) {
  __shared__ float red[4];
  const int64_t src = rows ? rows[blockIdx.x] : (int64_t)blockIdx.x;
  const float* xr = x + src * H;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) ss += xr[c] * xr[c];
  ss = block_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += blockDim.x) stf(out + (int64_t)blockIdx.x * H + c, xr[c] * r * w[c]);
}

// src[t] >= 0: row of x; -1: zeros; <= -2: state slot -(src + 2). save (optional, one entry per
// row): slot that takes this row's x afterwards. Only valid when every row is the single token of
// its sequence (then the row that reads a slot is the row that writes it, element by element in
// one thread); steps with longer portions save with shift_save after this kernel.
template <typename T>
__global__ void __launch_bounds__(256) token_shift_kernel(T* __restrict__ h, const float* __restrict__ x,
                                                          const float* __restrict__ mu, const int32_t* __restrict__ src,
                                                          float* __restrict__ state, const int32_t* __restrict__ save,
                                                          int H) {
  const int64_t row = blockIdx.x;
  const int s = src[row];
  const float* prev = s >= 0 ? x + (int64_t)s * H : (s == -1 ? nullptr : state + (int64_t)(-(s + 2)) * H);
  const int sv = save ? save[row] : -1;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float v = x[row * H + c];
    const float p = prev ? prev[c] : 0.f;
    stf(h + row * H + c, v + (p - v) * mu[c]);
    if (sv >= 0) state[(int64_t)sv * H + c] = v;
  }
}

__global__ void __launch_bounds__(256) shift_save_kernel(float* __restrict__ state, const float* __restrict__ x,
                                                         const int32_t* __restrict__ last_row,
                                                         const int32_t* __restrict__ slot, int H) {
  const int s = slot[blockIdx.x], r = last_row[blockIdx.x];
  if (s < 0 || r < 0) return;
  for (int c = threadIdx.x; c < H; c += blockDim.x) state[(int64_t)s * H + c] = x[(int64_t)r * H + c];
}

__device__ __forceinline__ float gelu_tanh_exact(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void __launch_bounds__(256) glu_gelu_tanh_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                            int64_t T_rows, int F) {
  const int64_t total = T_rows * F;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / F;
    const int c = (int)(i - t * F);
    stf(out + i, gelu_tanh_exact(ldf(in + t * 2 * F + c)) * ldf(in + t * 2 * F + F + c));
  }
}

template <typename T>
__global__ void __launch_bounds__(256) embed_rows_kernel(float* __restrict__ x, const int32_t* __restrict__ ids,
                                                         const T* __restrict__ embed, float scale, int H, int vocab) {
  const int64_t row = blockIdx.x;
  int id = ids[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // padding rows of a captured step
  for (int c = threadIdx.x; c < H; c += blockDim.x) x[row * H + c] = ldf(embed + (int64_t)id * H + c) * scale;
}

// ws / nws: 1 when the weight has H elements, 0 when it is a single gain. Three passes over the
// row: statistic of y, residual sum with the statistic of the new x, the next norm's output.
template <typename T>
__global__ void __launch_bounds__(256) rmsnorm_residual_next_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                    int64_t y_stride, const float* __restrict__ w,
                                                                    int ws, const float* __restrict__ nw, int nws,
                                                                    float eps, int H, T* __restrict__ out) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float* xr = x + row * H;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float v = ldf(yr + c);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float v = xr[c] + ldf(yr + c) * r * w[c * ws];
    xr[c] = v;
    s2 += v * v;
  }
  s2 = block_sum(s2, red);
  const float r2 = 1.0f / sqrtf(s2 / (float)H + eps);
  // each thread re-reads only the columns it wrote itself
  for (int c = threadIdx.x; c < H; c += blockDim.x) stf(out + row * H + c, xr[c] * r2 * nw[c * nws]);
}

template <typename T>
__global__ void __launch_bounds__(256) relu_sq_kernel(T* __restrict__ out, const T* __restrict__ in, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const float v = fmaxf(ldf(in + i), 0.f);
    stf(out + i, v * v);
  }
}

__global__ void __launch_bounds__(256) relu_sq_bf16x8_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ in,
                                                             int64_t n8) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    const u16x8 v = load8(in + i * 8);
    u16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float f = fmaxf(bf2f(v[j]), 0.f);
      o[j] = f2bf(f * f);
    }
    store8(out + i * 8, o);
  }
}

// Two passes over the row: residual sum with the statistic of the new x, then the norm's output
// (each thread re-reads only the columns it wrote itself). out == nullptr: the sum only.
template <typename T>
__global__ void __launch_bounds__(256) residual_add_rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                   int64_t y_stride, const float* __restrict__ w,
                                                                   float eps, int H, T* __restrict__ out) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float* xr = x + row * H;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float v = xr[c] + ldf(yr + c);
    xr[c] = v;
    ss += v * v;
  }
  if (!out) return;
  ss = block_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += blockDim.x) stf(out + row * H + c, xr[c] * r * w[c]);
}

template <typename T>
__global__ void __launch_bounds__(256) clamped_glu_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                          int64_t in_stride, int64_t T_rows, int F, float limit,
                                                          float alpha, int gate_col, float shift) {
  const int64_t total = T_rows * F;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / F;
    const int c = (int)(i - t * F);
    const T* r = in + t * in_stride;
    const float g = fminf(ldf(r + c), limit);
    const float u = fminf(fmaxf(ldf(r + F + c), -limit), limit);
    float v = g / (1.0f + expf(-alpha * g)) * (u + shift);
    if (gate_col >= 0) v *= 1.0f / (1.0f + expf(-ldf(r + gate_col)));
    stf(out + i, v);
  }
}

// bf16 rows with F % 8 == 0 and 16-byte aligned rows: 8 gates and 8 ups per thread
__global__ void __launch_bounds__(256) clamped_glu_bf16x8_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ in,
                                                                 int64_t in_stride, int64_t T_rows, int F8, float limit,
                                                                 float alpha, int gate_col, float shift) {
  const int64_t total = T_rows * F8;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / F8;
    const int c = (int)(i - t * F8) * 8;
    const uint16_t* r = in + t * in_stride;
    const u16x8 g8 = load8(r + c), u8 = load8(r + 8 * F8 + c);
    const float rg = gate_col >= 0 ? 1.0f / (1.0f + expf(-bf2f(r[gate_col]))) : 1.0f;
    u16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float g = fminf(bf2f(g8[j]), limit);
      const float u = fminf(fmaxf(bf2f(u8[j]), -limit), limit);
      o[j] = f2bf(g / (1.0f + expf(-alpha * g)) * (u + shift) * rg);
    }
    store8(out + t * 8 * F8 + c, o);
  }
}

__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ z, int64_t n, float cap, float inv) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    z[i] = cap * tanhf(z[i] * inv);
}

// one wave per (row, group)
// w_groups: groups per row when every column has its own weight (else 0: gs weights shared by
// the groups); gate: rows [groups * gs] of the output type with stride g_stride, sigmoid applied
template <typename T>
__global__ void __launch_bounds__(256) group_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                            const float* __restrict__ w, int64_t n_groups, int gs,
                                                            float eps, int groups, int w_full,
                                                            const T* __restrict__ gate, int64_t g_stride, int pair) {
  const int64_t g = blockIdx.x * (int64_t)(blockDim.x >> 6) + (threadIdx.x >> 6);
  if (g >= n_groups) return;
  const int lane = threadIdx.x & 63;
  const float* xr = x + g * gs;
  const int64_t row = g / groups;
  const int hg = (int)(g - row * groups);
  const float* wr = w_full ? w + (int64_t)hg * gs : w;
  const T* gr = gate ? gate + row * g_stride + (int64_t)hg * gs : nullptr;
  float ss = 0.f;
  if (pair) {   // gs even, 8-byte aligned fp32 rows: two neighbouring elements per lane
    for (int c = 2 * lane; c < gs; c += 128) {
      const float2 v = *reinterpret_cast<const float2*>(xr + c);
      ss += v.x * v.x + v.y * v.y;
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int c = 2 * lane; c < gs; c += 128) {
      const float2 v = *reinterpret_cast<const float2*>(xr + c);
      float a = v.x * r * wr[c], b = v.y * r * wr[c + 1];
      if (gr) {
        a *= 1.0f / (1.0f + expf(-ldf(gr + c)));
        b *= 1.0f / (1.0f + expf(-ldf(gr + c + 1)));
      }
      stf(out + g * gs + c, a);
      stf(out + g * gs + c + 1, b);
    }
    return;
  }
  for (int c = lane; c < gs; c += 64) ss += xr[c] * xr[c];
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)gs + eps);
  for (int c = lane; c < gs; c += 64) {
    float v = xr[c] * r * wr[c];
    if (gr) v *= 1.0f / (1.0f + expf(-ldf(gr + c)));
    stf(out + g * gs + c, v);
  }
}

// groups of gs % 4 == 0 columns, 16-byte aligned fp32 rows, 8-byte aligned outputs and gates: half a
// wave per (row, group), four neighbouring elements per lane (16-byte loads of x and w, 8-byte
// loads of the gate and stores); the sum of squares is reduced inside the half wave
__global__ void __launch_bounds__(256) group_rmsnorm_bf16x4_kernel(uint16_t* __restrict__ out, const float* __restrict__ x,
                                                                   const float* __restrict__ w, int64_t n_groups, int gs,
                                                                   float eps, int groups, int w_full,
                                                                   const uint16_t* __restrict__ gate, int64_t g_stride) {
  const int64_t g = blockIdx.x * (int64_t)(blockDim.x >> 5) + (threadIdx.x >> 5);
  const bool live = g < n_groups;
  const int sub = threadIdx.x & 31;
  const int64_t gg = live ? g : 0;
  const float* xr = x + gg * gs;
  const int64_t row = gg / groups;
  const int hg = (int)(gg - row * groups);
  const float* wr = w_full ? w + (int64_t)hg * gs : w;
  const uint16_t* gr = gate ? gate + row * g_stride + (int64_t)hg * gs : nullptr;
  float ss = 0.f;
  for (int c = 4 * sub; c < gs; c += 128) {
    const float4 v = *reinterpret_cast<const float4*>(xr + c);
    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
  }
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);   // stays inside the half wave
  if (!live) return;
  const float r = 1.0f / sqrtf(ss / (float)gs + eps);
  for (int c = 4 * sub; c < gs; c += 128) {
    const float4 v = *reinterpret_cast<const float4*>(xr + c), ww = *reinterpret_cast<const float4*>(wr + c);
    float y[4] = {v.x * r * ww.x, v.y * r * ww.y, v.z * r * ww.z, v.w * r * ww.w};
    if (gr) {
      const u16x4 g4 = *reinterpret_cast<const u16x4*>(gr + c);
#pragma unroll
      for (int q = 0; q < 4; ++q) y[q] *= __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * bf2f(g4[q])));
    }
    u16x4 o4;
#pragma unroll
    for (int q = 0; q < 4; ++q) o4[q] = f2bf(y[q]);
    *reinterpret_cast<u16x4*>(out + gg * gs + c) = o4;
  }
}

// ---- dynamic tanh in place of a norm: tanh(alpha x) * w + b, no statistics
// rows: gather (nullptr: all rows)
template <typename T>
__global__ void __launch_bounds__(256) dyt_norm_kernel(T* __restrict__ out, const float* __restrict__ x, float alpha,
                                                       const float* __restrict__ w, const float* __restrict__ b,
                                                       const int64_t* __restrict__ rows, int H) {
  const int64_t r = blockIdx.x;
  const float* xr = x + (rows ? rows[r] : r) * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) stf(out + r * H + c, tanhf(alpha * xr[c]) * w[c] + b[c]);
}

// x += (y1 + y2 + bias) (fp32 sums), or x = y1 (assign); out = tanh(alpha x) * w + b
template <typename T>
__global__ void __launch_bounds__(256) residual_dyt_kernel(float* __restrict__ x, const T* __restrict__ y1, int64_t s1,
                                                           const T* __restrict__ y2, int64_t s2,
                                                           const float* __restrict__ bias, float alpha,
                                                           const float* __restrict__ w, const float* __restrict__ b,
                                                           T* __restrict__ out, int H, int assign) {
  const int64_t r = blockIdx.x;
  float* xr = x + r * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    float y = ldf(y1 + r * s1 + c);
    if (y2) y += ldf(y2 + r * s2 + c);
    if (bias) y += bias[c];
    const float v = assign ? y : xr[c] + y;
    xr[c] = v;
    if (out) stf(out + r * H + c, tanhf(alpha * v) * w[c] + b[c]);
  }
}

// tanh on the hardware exp2 and reciprocal: for results that are rounded to bf16
__device__ __forceinline__ float tanh_hw(float x) {
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(2.8853900817779268f * x));
}

// bf16 rows with H % 4 == 0 and 8-byte aligned rows: 4 elements per thread, 16-byte accesses to
// the fp32 stream and the fp32 vectors
__global__ void __launch_bounds__(256) residual_dyt_bf16x4_kernel(float* __restrict__ x, const uint16_t* __restrict__ y1,
                                                                  int64_t s1, const uint16_t* __restrict__ y2, int64_t s2,
                                                                  const float* __restrict__ bias, float alpha,
                                                                  const float* __restrict__ w, const float* __restrict__ b,
                                                                  uint16_t* __restrict__ out, int64_t T_rows, int H4,
                                                                  int assign) {
  const int64_t total = T_rows * H4;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / H4;
    const int c = (int)(i - r * H4) * 4;
    const u16x4 a = *reinterpret_cast<const u16x4*>(y1 + r * s1 + c);
    float y[4] = {bf2f(a[0]), bf2f(a[1]), bf2f(a[2]), bf2f(a[3])};
    if (y2) {
      const u16x4 a2 = *reinterpret_cast<const u16x4*>(y2 + r * s2 + c);
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] += bf2f(a2[j]);
    }
    if (bias) {
      const float4 bb = *reinterpret_cast<const float4*>(bias + c);
      y[0] += bb.x, y[1] += bb.y, y[2] += bb.z, y[3] += bb.w;
    }
    float4* xp = reinterpret_cast<float4*>(x + r * 4 * H4 + c);
    float4 v;
    if (assign) {
      v = make_float4(y[0], y[1], y[2], y[3]);
    } else {
      v = *xp;
      v.x += y[0], v.y += y[1], v.z += y[2], v.w += y[3];
    }
    *xp = v;
    if (out) {
      const float4 ww = *reinterpret_cast<const float4*>(w + c), bn = *reinterpret_cast<const float4*>(b + c);
      u16x4 o;
      o[0] = f2bf(tanh_hw(alpha * v.x) * ww.x + bn.x);
      o[1] = f2bf(tanh_hw(alpha * v.y) * ww.y + bn.y);
      o[2] = f2bf(tanh_hw(alpha * v.z) * ww.z + bn.z);
      o[3] = f2bf(tanh_hw(alpha * v.w) * ww.w + bn.w);
      *reinterpret_cast<u16x4*>(out + r * 4 * H4 + c) = o;
    }
  }
}

// out row = [a row | b row] in the activation type
template <typename T>
__global__ void __launch_bounds__(256) pack_pair_kernel(T* __restrict__ out, const float* __restrict__ a,
                                                        const float* __restrict__ b, int Ha, int Hb) {
  const int64_t r = blockIdx.x;
  T* o = out + r * (Ha + Hb);
  for (int c = threadIdx.x; c < Ha; c += blockDim.x) stf(o + c, a[r * Ha + c]);
  for (int c = threadIdx.x; c < Hb; c += blockDim.x) stf(o + Ha + c, b[r * Hb + c]);
}

// x = gelu_tanh(x + bias) in place, any width
template <typename T>
__global__ void __launch_bounds__(256) bias_gelu_tanh_kernel(T* __restrict__ x, const float* __restrict__ bias,
                                                             int64_t T_rows, int F) {
  const int64_t total = T_rows * F;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % F);
    const float z = ldf(x + i) + (bias ? bias[c] : 0.f);
    stf(x + i, 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))));
  }
}

// bf16 rows with F % 8 == 0: 8 elements per thread
// (a workgroup takes RB whole rows: 32-bit index arithmetic, the bias row stays in cache)
__global__ void __launch_bounds__(256) bias_gelu_tanh_bf16x8_kernel(uint16_t* __restrict__ x, const float* __restrict__ bias,
                                                                    int64_t T_rows, int F8, int RB) {
  const int64_t r0 = (int64_t)blockIdx.x * RB;
  const int rows = (int)(T_rows - r0 < RB ? T_rows - r0 : RB);
  uint16_t* xb = x + r0 * 8 * F8;
  for (int i = threadIdx.x; i < rows * F8; i += blockDim.x) {
    const int c = (i % F8) * 8;
    float bz[8];
    if (bias) {
      const float4 b0 = *reinterpret_cast<const float4*>(bias + c), b1 = *reinterpret_cast<const float4*>(bias + c + 4);
      bz[0] = b0.x, bz[1] = b0.y, bz[2] = b0.z, bz[3] = b0.w, bz[4] = b1.x, bz[5] = b1.y, bz[6] = b1.z, bz[7] = b1.w;
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) bz[j] = 0.f;
    }
    const u16x8 v = load8(xb + (int64_t)i * 8);
    u16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float z = bf2f(v[j]) + bz[j];
      const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
      // 0.5 z (1 + tanh u) = z - z / (1 + e^(2u))
      o[j] = f2bf(z - z * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(2.8853900817779268f * u)));
    }
    store8(xb + (int64_t)i * 8, o);
  }
}

}  // namespace

void launch_embed_pos(float* x, const int32_t* ids, const int32_t* pos, const void* embed, const void* ptab,
                      int64_t T, int H, int vocab, int max_pos, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    embed_pos_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>(x, ids, pos, (const float*)embed,
                                                                  (const float*)ptab, H, vocab, max_pos);
  else
    embed_pos_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>(x, ids, pos, (const uint16_t*)embed,
                                                                     (const uint16_t*)ptab, H, vocab, max_pos);
}

void launch_rmsnorm_residual(float* x, const void* y, int64_t y_stride, const float* w, float eps, int64_t T, int H,
                             void* cast_out, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    rmsnorm_residual_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const float*)y, y_stride, w, eps, H,
                                                                         (float*)cast_out);
  else
    rmsnorm_residual_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const uint16_t*)y, y_stride, w, eps,
                                                                            H, (uint16_t*)cast_out);
}

void launch_rmsnorm_f32(void* out, const float* x, const int64_t* rows, const float* w, float eps, int64_t T, int H,
                        bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    rmsnorm_f32_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>((float*)out, x, rows, w, eps, H);
  else
    rmsnorm_f32_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)out, x, rows, w, eps, H);
}

void launch_token_shift(void* h, const float* x, const float* mu, const int32_t* src, float* state,
                        const int32_t* save, int64_t T, int H, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    token_shift_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>((float*)h, x, mu, src, state, save, H);
  else
    token_shift_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)h, x, mu, src, state, save, H);
}

void launch_shift_save(float* state, const float* x, const int32_t* last_row, const int32_t* slot, int n, int H,
                       hipStream_t stream) {
  if (n == 0) return;
  shift_save_kernel<<<dim3((unsigned)n), 256, 0, stream>>>(state, x, last_row, slot, H);
}

void launch_glu_gelu_tanh(void* out, const void* in, int64_t T, int F, bool f32, hipStream_t stream) {
  if (T == 0 || F == 0) return;
  int64_t g = (T * F + 255) / 256;
  if (g > 8192) g = 8192;
  if (f32)
    glu_gelu_tanh_kernel<float><<<dim3((unsigned)g), 256, 0, stream>>>((float*)out, (const float*)in, T, F);
  else
    glu_gelu_tanh_kernel<uint16_t><<<dim3((unsigned)g), 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)in, T, F);
}

void launch_embed_rows(float* x, const int32_t* ids, const void* embed, float scale, int64_t T, int H, int vocab,
                       bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    embed_rows_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>(x, ids, (const float*)embed, scale, H, vocab);
  else
    embed_rows_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>(x, ids, (const uint16_t*)embed, scale, H, vocab);
}

void launch_rmsnorm_residual_next(float* x, const void* y, int64_t y_stride, const float* w, int w_n, const float* nw,
                                  int nw_n, float eps, int64_t T, int H, void* out, bool f32, hipStream_t stream) {
  if (T == 0) return;
  const int ws = w_n == 1 ? 0 : 1, nws = nw_n == 1 ? 0 : 1;
  if (f32)
    rmsnorm_residual_next_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const float*)y, y_stride, w, ws, nw,
                                                                              nws, eps, H, (float*)out);
  else
    rmsnorm_residual_next_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const uint16_t*)y, y_stride, w,
                                                                                 ws, nw, nws, eps, H, (uint16_t*)out);
}

void launch_relu_sq(void* out, const void* in, int64_t n, bool f32, hipStream_t stream) {
  if (n == 0) return;
  if (!f32 && n % 8 == 0) {
    int64_t g = (n / 8 + 255) / 256;
    if (g > 16384) g = 16384;
    relu_sq_bf16x8_kernel<<<dim3((unsigned)g), 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)in, n / 8);
    return;
  }
  int64_t g = (n + 255) / 256;
  if (g > 16384) g = 16384;
  if (f32)
    relu_sq_kernel<float><<<dim3((unsigned)g), 256, 0, stream>>>((float*)out, (const float*)in, n);
  else
    relu_sq_kernel<uint16_t><<<dim3((unsigned)g), 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)in, n);
}

void launch_softcap(float* z, int64_t n, float cap, float scale, hipStream_t stream) {
  if (n == 0) return;
  int64_t g = (n + 255) / 256;
  if (g > 16384) g = 16384;
  softcap_kernel<<<dim3((unsigned)g), 256, 0, stream>>>(z, n, cap, scale / cap);
}

void launch_residual_add_rmsnorm(float* x, const void* y, int64_t y_stride, const float* w, float eps, int64_t T, int H,
                                 void* out, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    residual_add_rmsnorm_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const float*)y, y_stride, w, eps, H,
                                                                             (float*)out);
  else
    residual_add_rmsnorm_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const uint16_t*)y, y_stride, w, eps,
                                                                                H, (uint16_t*)out);
}

void launch_clamped_glu(void* out, const void* in, int64_t in_stride, int64_t T, int F, float limit, float alpha,
                        int gate_col, float shift, bool f32, hipStream_t stream) {
  if (T == 0 || F == 0) return;
  if (!f32 && F % 8 == 0 && in_stride % 8 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    int64_t g8 = (T * (F / 8) + 255) / 256;
    if (g8 > 16384) g8 = 16384;
    clamped_glu_bf16x8_kernel<<<dim3((unsigned)g8), 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)in, in_stride, T,
                                                                      F / 8, limit, alpha, gate_col, shift);
    return;
  }
  int64_t g = (T * F + 255) / 256;
  if (g > 8192) g = 8192;
  if (f32)
    clamped_glu_kernel<float><<<dim3((unsigned)g), 256, 0, stream>>>((float*)out, (const float*)in, in_stride, T, F,
                                                                    limit, alpha, gate_col, shift);
  else
    clamped_glu_kernel<uint16_t><<<dim3((unsigned)g), 256, 0, stream>>>((uint16_t*)out, (const uint16_t*)in, in_stride,
                                                                       T, F, limit, alpha, gate_col, shift);
}

void launch_group_rmsnorm(void* out, const float* x, const float* w, bool w_full, const void* gate, int64_t g_stride,
                          int64_t T, int groups, int gs, float eps, bool f32, hipStream_t stream) {
  const int64_t ng = T * groups;
  if (ng == 0) return;
  if (!f32 && gs % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)out % 8) == 0 &&
      (gate == nullptr || (g_stride % 4 == 0 && ((uintptr_t)gate % 8) == 0))) {
    group_rmsnorm_bf16x4_kernel<<<dim3((unsigned)((ng + 7) / 8)), 256, 0, stream>>>(
        (uint16_t*)out, x, w, ng, gs, eps, groups, w_full ? 1 : 0, (const uint16_t*)gate, g_stride);
    return;
  }
  const unsigned g = (unsigned)((ng + 3) / 4);
  const int pair = (gs % 2 == 0 && ((uintptr_t)x % 8) == 0) ? 1 : 0;
  if (f32)
    group_rmsnorm_kernel<float><<<dim3(g), 256, 0, stream>>>((float*)out, x, w, ng, gs, eps, groups, w_full ? 1 : 0,
                                                             (const float*)gate, g_stride, pair);
  else
    group_rmsnorm_kernel<uint16_t><<<dim3(g), 256, 0, stream>>>((uint16_t*)out, x, w, ng, gs, eps, groups, w_full ? 1 : 0,
                                                                (const uint16_t*)gate, g_stride, pair);
}

void launch_dyt_norm(void* out, const float* x, float alpha, const float* w, const float* b, const int64_t* rows,
                     int64_t n_out, int H, bool f32, hipStream_t stream) {
  if (n_out == 0) return;
  if (f32)
    dyt_norm_kernel<float><<<dim3((unsigned)n_out), 256, 0, stream>>>((float*)out, x, alpha, w, b, rows, H);
  else
    dyt_norm_kernel<uint16_t><<<dim3((unsigned)n_out), 256, 0, stream>>>((uint16_t*)out, x, alpha, w, b, rows, H);
}

void launch_residual_dyt(float* x, const void* y1, int64_t s1, const void* y2, int64_t s2, const float* bias, float alpha,
                         const float* w, const float* b, void* out, int64_t T, int H, bool assign, bool f32,
                         hipStream_t stream) {
  if (T == 0) return;
  auto al8 = [](const void* p) { return ((uintptr_t)p % 8) == 0; };
  if (!f32 && H % 4 == 0 && s1 % 4 == 0 && s2 % 4 == 0 && al8(y1) && al8(y2) && al8(out) && ((uintptr_t)x % 16) == 0 &&
      ((uintptr_t)bias % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)b % 16) == 0) {
    int64_t g = (T * (H / 4) + 255) / 256;
    if (g > 16384) g = 16384;
    residual_dyt_bf16x4_kernel<<<dim3((unsigned)g), 256, 0, stream>>>(x, (const uint16_t*)y1, s1, (const uint16_t*)y2, s2,
                                                                      bias, alpha, w, b, (uint16_t*)out, T, H / 4,
                                                                      assign ? 1 : 0);
    return;
  }
  if (f32)
    residual_dyt_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const float*)y1, s1, (const float*)y2, s2, bias,
                                                                     alpha, w, b, (float*)out, H, assign ? 1 : 0);
  else
    residual_dyt_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>(x, (const uint16_t*)y1, s1, (const uint16_t*)y2,
                                                                        s2, bias, alpha, w, b, (uint16_t*)out, H,
                                                                        assign ? 1 : 0);
}

void launch_pack_pair(void* out, const float* a, const float* b, int64_t T, int Ha, int Hb, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    pack_pair_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>((float*)out, a, b, Ha, Hb);
  else
    pack_pair_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)out, a, b, Ha, Hb);
}

void launch_bias_gelu_tanh(void* x, const float* bias, int64_t T, int F, bool f32, hipStream_t stream) {
  if (T == 0 || F == 0) return;
  if (!f32 && F % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)bias % 16) == 0) {
    const int F8 = F / 8;
    int RB = 2048 / F8;                      // about 8 vectors per thread
    RB = RB < 1 ? 1 : RB;
    bias_gelu_tanh_bf16x8_kernel<<<dim3((unsigned)((T + RB - 1) / RB)), 256, 0, stream>>>((uint16_t*)x, bias, T, F8, RB);
    return;
  }
  int64_t g = (T * F + 255) / 256;
  if (g > 8192) g = 8192;
  if (f32)
    bias_gelu_tanh_kernel<float><<<dim3((unsigned)g), 256, 0, stream>>>((float*)x, bias, T, F);
  else
    bias_gelu_tanh_kernel<uint16_t><<<dim3((unsigned)g), 256, 0, stream>>>((uint16_t*)x, bias, T, F);
}

}  // namespace nga
