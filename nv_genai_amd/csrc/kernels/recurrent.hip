// Gated linear recurrences with a matrix state per head, carried across steps in state slots.
//
//   hgrn2_scan   per head S <- diag(f) S + (1 - f) v^T, o = S^T q over the rows of a segment
//                (a prompt portion, or a single decode row), with q = silu(q_pre) and
//                f = lower + (1 - lower) * sigmoid(f_pre + f_bias) formed in fp32 in the kernel.
//
//   mlstm_scan   per head a matrix memory with exponential gates kept stable by a running maximum m:
//                m' = max(f + m, i), S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k,
//                o = S^T q / (max(|n . q|, e^(-m')) + 1e-6), with the log gates
//                i = cap tanh((i_pre + b) / cap), f = logsigmoid(cap tanh((f_pre + b) / cap)) and
//                q scaled by d^(-1/2), all formed in fp32 in the kernel. Same tiling as hgrn2_scan;
//                every value tile carries n and m itself (they do not depend on the value column)
//                and the state slot keeps one copy of (n, m) per 16 value columns: a tile reads the
//                copy of its first columns and writes the copies of its own columns, so no tile
//                reads what another tile of the launch writes. The gate chain of a pass (m, both
//                decays, e^(-m)) is a prefix scan over the lanes of the first wave, shared through LDS.
//
// A workgroup owns (segment, head, tile of VT value columns): thread (rg, j) keeps the state
// elements S[rg * NR + k][j] in registers for the whole segment, so the state is read from its
// slot once and written back once. Rows are staged through LDS TC at a time: the raw values of the
// next TC rows are loaded into registers before the current ones are processed, and the
// activations are applied on the way into LDS. Per row every thread reads its NR gates and
// queries as 16-byte LDS vectors, updates its NR state elements and adds its part of o; the RG
// parts are summed through LDS for all TC rows at once. The tile width VT is chosen by the host so
// that a launch has enough workgroups. State, gates and sums are fp32 whatever the activation type.
#include "common.h"
#include "kernels.h"

namespace nga {

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }

// 1 / (1 + 2^(-z log2 e)) on the hardware exp2 and reciprocal (1 ulp each): the activations are
// recomputed by every value tile of a head, so their cost is on the scan's critical path
__device__ __forceinline__ float sigmoid_fast(float z) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
}

constexpr int TC = 16;   // rows staged per pass

// proj row: [q_pre (H*d) | f_pre (H*d) | v (H*dv) | ...]. cu == nullptr: segment b is row b.
// Rows of a head are padded to DP = RG * NR in LDS (q = 0, f = 1: a padded state row stays 0).
template <typename T, int NR, int VT>
__global__ void __launch_bounds__(256) hgrn2_scan_kernel(float* __restrict__ out, const T* __restrict__ proj,
                                                         int64_t stride, const float* __restrict__ f_bias,
                                                         const float* __restrict__ lower, float* __restrict__ state,
                                                         int H, int d, int dv, const int32_t* __restrict__ cu,
                                                         const int32_t* __restrict__ slots,
                                                         const int32_t* __restrict__ pos) {
  constexpr int RG = 256 / VT;
  constexpr int DP = RG * NR;              // padded rows of a head
  constexpr int NQ = TC * DP / 256;        // q (and f) elements a thread stages per pass
  constexpr int NV = (TC * VT + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs[TC * DP];
  __shared__ __attribute__((aligned(16))) float fs[TC * DP];
  __shared__ float vs[TC * VT];
  __shared__ float part[TC * 256];
  const int vt = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int t0 = cu ? cu[b] : b, t1 = cu ? cu[b + 1] : b + 1;
  if (t1 <= t0) return;
  const int slot = slots[b];
  const bool fresh = slot < 0 || pos[t0] == 0;
  const int tid = threadIdx.x;
  const int j = tid % VT, rg = tid / VT;
  const int col = vt * VT + j;
  const bool colok = col < dv;
  float* sp = slot >= 0 ? state + ((int64_t)slot * H + h) * (int64_t)d * dv : nullptr;
  float S[NR];
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const int i = rg * NR + k;
    S[k] = (!fresh && colok && i < d) ? sp[(int64_t)i * dv + col] : 0.f;
  }
  const int qoff = h * d, foff = H * d + h * d, voff = 2 * H * d + h * dv + vt * VT;
  float rq[NQ], rf[NQ], rv[NV];
  // raw values of rows [tc, tc + TC) into registers (rows past t1 and padded columns: neutral)
  auto fetch = [&](int tc) {
#pragma unroll
    for (int x = 0; x < NQ; ++x) {
      const int e = tid + 256 * x, tt = e / DP, i = e % DP;
      const bool ok = tc + tt < t1 && i < d;
      const T* pr = proj + (int64_t)(tc + tt) * stride;
      rq[x] = ok ? ldf(pr + qoff + i) : 0.f;
      rf[x] = ok ? ldf(pr + foff + i) : 0.f;
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = tid + 256 * x, tt = e / VT, jj = e % VT;
      rv[x] = (e < TC * VT && tc + tt < t1 && vt * VT + jj < dv) ? ldf(proj + (int64_t)(tc + tt) * stride + voff + jj) : 0.f;
    }
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += TC) {
    const int nt = t1 - tc < TC ? t1 - tc : TC;
    __syncthreads();   // the previous pass is done with qs / fs / vs / part
#pragma unroll
    for (int x = 0; x < NQ; ++x) {
      const int e = tid + 256 * x, i = e % DP;
      if (i < d) {
        const float lw = lower[qoff + i];
        qs[e] = rq[x] * sigmoid_fast(rq[x]);
        fs[e] = lw + (1.0f - lw) * sigmoid_fast(rf[x] + f_bias[qoff + i]);
      } else {
        qs[e] = 0.f;
        fs[e] = 1.f;
      }
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = tid + 256 * x;
      if (e < TC * VT) vs[e] = rv[x];
    }
    __syncthreads();
    if (tc + TC < t1) fetch(tc + TC);   // lands while this pass computes
    auto row = [&](int tt) {
      const float vv = vs[tt * VT + j];
      const float4* fr = reinterpret_cast<const float4*>(fs + tt * DP + rg * NR);
      const float4* qr = reinterpret_cast<const float4*>(qs + tt * DP + rg * NR);
      float p = 0.f;
#pragma unroll
      for (int k4 = 0; k4 < NR / 4; ++k4) {
        const float4 f4 = fr[k4], q4 = qr[k4];
        const float fa[4] = {f4.x, f4.y, f4.z, f4.w}, qa[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int k = 4 * k4 + u;
          S[k] = fa[u] * S[k] + (1.0f - fa[u]) * vv;
          p += S[k] * qa[u];
        }
      }
      part[tt * 256 + tid] = p;
    };
    if (nt == TC) {   // full pass: unrolled, so the LDS reads of later rows run ahead of the recurrence
#pragma unroll
      for (int tt = 0; tt < TC; ++tt) row(tt);
    } else {
      for (int tt = 0; tt < nt; ++tt) row(tt);
    }
    __syncthreads();
    for (int e = tid; e < nt * VT; e += 256) {
      const int tt = e / VT, jj = e % VT;
      if (vt * VT + jj < dv) {
        float s2 = 0.f;
#pragma unroll
        for (int r = 0; r < RG; ++r) s2 += part[tt * 256 + r * VT + jj];
        out[(int64_t)(tc + tt) * H * dv + h * dv + vt * VT + jj] = s2;
      }
    }
  }
  if (sp && colok) {
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const int i = rg * NR + k;
      if (i < d) sp[(int64_t)i * dv + col] = S[k];
    }
  }
}

template <typename T, int VT>
bool launch_hgrn2_vt(float* out, const T* proj, int64_t stride, const float* f_bias, const float* lower, float* state,
                     int H, int d, int dv, const int32_t* cu, const int32_t* slots, const int32_t* pos, int n_seg,
                     hipStream_t stream) {
  constexpr int RG = 256 / VT;
  const int nr = (d + RG - 1) / RG;
  const dim3 grid((unsigned)((dv + VT - 1) / VT), (unsigned)H, (unsigned)n_seg);
#define NGA_HGRN2_CASE(N)                                                                                            \
  if (nr <= N) {                                                                                                     \
    hgrn2_scan_kernel<T, N, VT><<<grid, 256, 0, stream>>>(out, proj, stride, f_bias, lower, state, H, d, dv, cu, slots, \
                                                          pos);                                                      \
    return true;                                                                                                     \
  }
  // at most 256 padded rows per head in LDS: NR <= 64 / 32 / 16 for tiles of 64 / 32 / 16 columns
  NGA_HGRN2_CASE(4)
  NGA_HGRN2_CASE(8)
  NGA_HGRN2_CASE(16)
  if constexpr (VT >= 32) {
    NGA_HGRN2_CASE(32)
  }
  if constexpr (VT >= 64) {
    NGA_HGRN2_CASE(64)
  }
#undef NGA_HGRN2_CASE
  return false;
}

// The widest value tile that still gives about four workgroups per CU; narrower tiles when the
// key size needs more row groups than a wide tile leaves.
template <typename T>
bool launch_hgrn2_t(float* out, const T* proj, int64_t stride, const float* f_bias, const float* lower, float* state,
                    int H, int d, int dv, const int32_t* cu, const int32_t* slots, const int32_t* pos, int n_seg,
                    hipStream_t stream) {
  const int64_t base = (int64_t)n_seg * H;
  int vt = dv <= 16 ? 16 : (dv <= 32 ? 32 : 64);
  while (vt > 16 && base * ((dv + vt - 1) / vt) < 1024) vt /= 2;
#define NGA_HGRN2_ARGS out, proj, stride, f_bias, lower, state, H, d, dv, cu, slots, pos, n_seg, stream
  if (vt == 64 && launch_hgrn2_vt<T, 64>(NGA_HGRN2_ARGS)) return true;
  if (vt >= 32 && launch_hgrn2_vt<T, 32>(NGA_HGRN2_ARGS)) return true;
  return launch_hgrn2_vt<T, 16>(NGA_HGRN2_ARGS);
#undef NGA_HGRN2_ARGS
}


// ---------------------------------------------------------------------------------------------
// mLSTM. proj row: q [H*d] at q_off, k [H*d] at k_off, v [H*dv] at v_off, gate pre-activations
// [i (H) | f (H)] at g_off. State slot of a head: S [d][dv], then ceil(dv / 16) copies of (n [d], m).
// cu == nullptr: segment b is row b. Padded state rows (i >= d) see k = q = 0 and stay 0.
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// The gate functions of the scan, all in fp32. PRECISE (fp32 activations): the library functions.
// Otherwise (bf16 activations) the same formulas on the hardware exp2 / log2 / reciprocal (about
// 1 ulp each): the gate phase of a pass is a serial stretch in which three of the four waves wait.
template <bool PRECISE> struct GateMath;
template <> struct GateMath<true> {
  static __device__ __forceinline__ float exp(float x) { return expf(x); }
  static __device__ __forceinline__ float tanh(float x) { return tanhf(x); }
  static __device__ __forceinline__ float logsig(float z) { return log_sigmoid(z); }
};
template <> struct GateMath<false> {
  static __device__ __forceinline__ float exp(float x) { return __builtin_amdgcn_exp2f(1.4426950408889634f * x); }
  static __device__ __forceinline__ float tanh(float x) {
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(2.8853900817779268f * x));
  }
  // min(z, 0) - ln(1 + e^(-|z|)); the sum 1 + e^(-|z|) lies in (1, 2], so the logarithm loses nothing
  static __device__ __forceinline__ float logsig(float z) {
    const float e = __builtin_amdgcn_exp2f(-1.4426950408889634f * fabsf(z));
    return fminf(z, 0.f) - 0.6931471805599453f * __builtin_amdgcn_logf(1.0f + e);
  }
};

// TCN: rows staged per pass (16 for prompt portions; 1 for launches whose segments are single rows: a
// sixteenth of the LDS, so that all workgroups of a decode step are resident at once)
template <typename T, int NR, int VT, int TCN>
__global__ void __launch_bounds__(256) mlstm_scan_kernel(float* __restrict__ out, const T* __restrict__ proj,
                                                         int64_t stride, const float* __restrict__ gate_bias,
                                                         float* __restrict__ state, int H, int d, int dv, float cap,
                                                         const int32_t* __restrict__ cu,
                                                         const int32_t* __restrict__ slots,
                                                         const int32_t* __restrict__ pos, int q_off, int k_off,
                                                         int v_off, int g_off) {
  using GM = GateMath<sizeof(T) == 4>;
  constexpr int RG = 256 / VT;
  constexpr int DP = RG * NR;              // padded rows of a head
  constexpr int NQ = (TCN * DP + 255) / 256;   // q (and k) elements a thread stages per pass
  constexpr int NV = (TCN * VT + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs[TCN * DP];
  __shared__ __attribute__((aligned(16))) float ks[TCN * DP];
  __shared__ float vs[TCN * VT];
  __shared__ float part[TCN * 256];
  __shared__ float partn[TCN * RG];
  __shared__ float ga[TCN], gb[TCN], gem[TCN];   // decay of the old state, weight of the new row, e^(-m)
  __shared__ float m_carry;
  const int vt = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int t0 = cu ? cu[b] : b, t1 = cu ? cu[b + 1] : b + 1;
  if (t1 <= t0) return;
  const int slot = slots[b];
  const bool fresh = slot < 0 || pos[t0] == 0;
  const int tid = threadIdx.x;
  const int j = tid % VT, rg = tid / VT;
  const int col = vt * VT + j;
  const bool colok = col < dv;
  const int ncopy = (dv + 15) / 16;        // copies of (n, m): one per 16 value columns
  const int64_t ssz = (int64_t)d * dv + (int64_t)ncopy * (d + 1);
  float* sp = slot >= 0 ? state + ((int64_t)slot * H + h) * ssz : nullptr;
  // this tile reads the copy of its first 16 columns and writes the copies of all its columns: no
  // tile reads what another tile of the launch writes, whatever tile widths the launches use
  const int c0 = vt * (VT / 16), c1 = min(ncopy, (vt + 1) * (VT / 16));
  const float* nm_in = sp ? sp + (int64_t)d * dv + (int64_t)c0 * (d + 1) : nullptr;
  float S[NR], n[NR];
  // n goes through LDS: one global access per element and workgroup instead of one per thread
  if (!fresh && tid < d) part[tid] = nm_in[tid];
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const int i = rg * NR + k;
    const bool ld = !fresh && i < d;
    S[k] = (ld && colok) ? sp[(int64_t)i * dv + col] : 0.f;
    n[k] = ld ? part[i] : 0.f;
  }
  if (tid == 0) m_carry = fresh ? 0.f : nm_in[d];
  const float qscale = 1.0f / sqrtf((float)d);
  const float inv_cap = 1.0f / cap;
  const int qo = q_off + h * d, ko = k_off + h * d, vo = v_off + h * dv + vt * VT;
  float rq[NQ], rk[NQ], rv[NV], ri = 0.f, rf = 0.f;
  // raw values of rows [tc, tc + TCN) into registers (rows past t1 and padded columns: zeros)
  auto fetch = [&](int tc) {
#pragma unroll
    for (int x = 0; x < NQ; ++x) {
      const int e = tid + 256 * x, tt = e / DP, i = e % DP;
      const bool ok = e < TCN * DP && tc + tt < t1 && i < d;
      const T* pr = proj + (int64_t)(tc + tt) * stride;
      rq[x] = ok ? ldf(pr + qo + i) : 0.f;
      rk[x] = ok ? ldf(pr + ko + i) : 0.f;
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = tid + 256 * x, tt = e / VT, jj = e % VT;
      rv[x] = (e < TCN * VT && tc + tt < t1 && vt * VT + jj < dv) ? ldf(proj + (int64_t)(tc + tt) * stride + vo + jj) : 0.f;
    }
    if (tid < TCN && tc + tid < t1) {
      const T* pr = proj + (int64_t)(tc + tid) * stride + g_off;
      ri = ldf(pr + h);
      rf = ldf(pr + H + h);
    }
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += TCN) {
    const int nt = t1 - tc < TCN ? t1 - tc : TCN;
    __syncthreads();   // the previous pass is done with the staged rows, part / partn and the gate chain
#pragma unroll
    for (int x = 0; x < NQ; ++x) {
      const int e = tid + 256 * x;
      if (e < TCN * DP) {
        qs[e] = rq[x] * qscale;
        ks[e] = rk[x];
      }
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int e = tid + 256 * x;
      if (e < TCN * VT) vs[e] = rv[x];
    }
    if (tid < 64) {   // the gate chain of the pass on the first wave, one row per lane, straight from the
      // lane's registers: the running maximum m_t = max(f_t + m_(t-1), i_t) is a prefix scan over the
      // maps m -> max(m + A, B), composed as (A1, B1) then (A2, B2) = (A1 + A2, max(B1 + A2, B2));
      // lanes past the pass's rows hold the identity. The three exponentials of all rows are then
      // taken side by side.
      float A = 0.f, B = -INFINITY;
      if (tid < nt) {
        B = cap * GM::tanh((ri + gate_bias[h]) * inv_cap);
        A = GM::logsig(cap * GM::tanh((rf + gate_bias[H + h]) * inv_cap));
      }
      const float f_t = A, i_t = B;
#pragma unroll
      for (int o = 1; o < TCN; o <<= 1) {
        const float Ap = __shfl_up(A, o, 64), Bp = __shfl_up(B, o, 64);
        if (tid >= o) {
          B = fmaxf(Bp + A, B);
          A = Ap + A;
        }
      }
      const float m0 = m_carry;
      const float m = fmaxf(m0 + A, B);
      float mp = __shfl_up(m, 1, 64);
      if (tid == 0) mp = m0;
      if (tid < nt) {
        ga[tid] = GM::exp(f_t + mp - m);
        gb[tid] = GM::exp(i_t - m);
        gem[tid] = GM::exp(-m);
      }
      if (tid == TCN - 1) m_carry = m;      // (lanes past nt pass the last row's maximum on)
    }
    __syncthreads();
    if (tc + TCN < t1) fetch(tc + TCN);   // lands while this pass computes
    auto row = [&](int tt) {
      const float a = ga[tt];
      const float bv = gb[tt] * vs[tt * VT + j], bb = gb[tt];
      const float4* kr = reinterpret_cast<const float4*>(ks + tt * DP + rg * NR);
      const float4* qr = reinterpret_cast<const float4*>(qs + tt * DP + rg * NR);
      float p = 0.f, pn = 0.f;
#pragma unroll
      for (int k4 = 0; k4 < NR / 4; ++k4) {
        const float4 k4v = kr[k4], q4 = qr[k4];
        const float ka[4] = {k4v.x, k4v.y, k4v.z, k4v.w}, qa[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int k = 4 * k4 + u;
          S[k] = a * S[k] + ka[u] * bv;
          n[k] = a * n[k] + ka[u] * bb;
          p += S[k] * qa[u];
          pn += n[k] * qa[u];
        }
      }
      part[tt * 256 + tid] = p;
      if (j == 0) partn[tt * RG + rg] = pn;
    };
    if (nt == TCN) {   // full pass: unrolled, so the LDS reads of later rows run ahead of the recurrence
#pragma unroll
      for (int tt = 0; tt < TCN; ++tt) row(tt);
    } else {
      for (int tt = 0; tt < nt; ++tt) row(tt);
    }
    __syncthreads();
    for (int e = tid; e < nt * VT; e += 256) {
      const int tt = e / VT, jj = e % VT;
      if (vt * VT + jj < dv) {
        float s2 = 0.f, nq = 0.f;
#pragma unroll
        for (int r = 0; r < RG; ++r) {
          s2 += part[tt * 256 + r * VT + jj];
          nq += partn[tt * RG + r];
        }
        out[(int64_t)(tc + tt) * H * dv + h * dv + vt * VT + jj] = s2 / (fmaxf(fabsf(nq), gem[tt]) + 1e-6f);
      }
    }
  }
  if (sp) {
    __syncthreads();   // m_carry of the last pass; the last pass is done with part
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const int i = rg * NR + k;
      if (i < d && colok) sp[(int64_t)i * dv + col] = S[k];
      if (j == 0) part[i] = n[k];
    }
    __syncthreads();
    for (int e = tid; e < (c1 - c0) * d; e += 256) {   // the copies of n this tile owns
      const int c = e / d, i = e - c * d;
      sp[(int64_t)d * dv + (int64_t)(c0 + c) * (d + 1) + i] = part[i];
    }
    if (tid < c1 - c0) sp[(int64_t)d * dv + (int64_t)(c0 + tid) * (d + 1) + d] = m_carry;
  }
}

template <typename T, int VT, int TCN>
bool launch_mlstm_vt(float* out, const T* proj, int64_t stride, const float* gate_bias, float* state, int H, int d,
                     int dv, float cap, const int32_t* cu, const int32_t* slots, const int32_t* pos, int n_seg, int q_off,
                     int k_off, int v_off, int g_off, hipStream_t stream) {
  constexpr int RG = 256 / VT;
  const int nr = (d + RG - 1) / RG;
  const dim3 grid((unsigned)((dv + VT - 1) / VT), (unsigned)H, (unsigned)n_seg);
#define NGA_MLSTM_CASE(N)                                                                                            \
  if (nr <= N) {                                                                                                     \
    mlstm_scan_kernel<T, N, VT, TCN><<<grid, 256, 0, stream>>>(out, proj, stride, gate_bias, state, H, d, dv, cap, cu, \
                                                               slots, pos, q_off, k_off, v_off, g_off);              \
    return true;                                                                                                     \
  }
  // at most 256 padded rows per head in LDS: NR <= 64 / 32 / 16 for tiles of 64 / 32 / 16 columns
  NGA_MLSTM_CASE(4)
  NGA_MLSTM_CASE(8)
  NGA_MLSTM_CASE(16)
  if constexpr (VT >= 32) {
    NGA_MLSTM_CASE(32)
  }
  if constexpr (VT >= 64) {
    NGA_MLSTM_CASE(64)
  }
#undef NGA_MLSTM_CASE
  return false;
}

template <typename T>
bool launch_mlstm_t(float* out, const T* proj, int64_t stride, const float* gate_bias, float* state, int H, int d, int dv,
                    float cap, const int32_t* cu, const int32_t* slots, const int32_t* pos, int n_seg, int q_off,
                    int k_off, int v_off, int g_off, hipStream_t stream) {
  const int64_t base = (int64_t)n_seg * H;
  int vt = dv <= 16 ? 16 : (dv <= 32 ? 32 : 64);
  while (vt > 16 && base * ((dv + vt - 1) / vt) < 1024) vt /= 2;
#define NGA_MLSTM_ARGS out, proj, stride, gate_bias, state, H, d, dv, cap, cu, slots, pos, n_seg, q_off, k_off, v_off, g_off, stream
  if (cu == nullptr) {   // every segment is one row: one row staged per pass
    if (vt == 64 && launch_mlstm_vt<T, 64, 1>(NGA_MLSTM_ARGS)) return true;
    if (vt >= 32 && launch_mlstm_vt<T, 32, 1>(NGA_MLSTM_ARGS)) return true;
    return launch_mlstm_vt<T, 16, 1>(NGA_MLSTM_ARGS);
  }
  if (vt == 64 && launch_mlstm_vt<T, 64, TC>(NGA_MLSTM_ARGS)) return true;
  if (vt >= 32 && launch_mlstm_vt<T, 32, TC>(NGA_MLSTM_ARGS)) return true;
  return launch_mlstm_vt<T, 16, TC>(NGA_MLSTM_ARGS);
#undef NGA_MLSTM_ARGS
}

}  // namespace

int mlstm_max_dim() { return 256; }   // padded rows of a head that fit the LDS staging

bool launch_mlstm_scan(float* out, const void* proj, int64_t stride, const float* gate_bias, float* state, int H, int d,
                       int dv, float cap, const int32_t* cu, const int32_t* slots, const int32_t* pos, int n_seg,
                       int q_off, int k_off, int v_off, int g_off, bool f32, hipStream_t stream) {
  if (n_seg == 0) return true;
  if (f32)
    return launch_mlstm_t<float>(out, (const float*)proj, stride, gate_bias, state, H, d, dv, cap, cu, slots, pos, n_seg,
                                 q_off, k_off, v_off, g_off, stream);
  return launch_mlstm_t<uint16_t>(out, (const uint16_t*)proj, stride, gate_bias, state, H, d, dv, cap, cu, slots, pos,
                                  n_seg, q_off, k_off, v_off, g_off, stream);
}

int hgrn2_max_dim(int dv) { return 256; }   // padded rows of a head that fit the LDS staging

bool launch_hgrn2_scan(float* out, const void* proj, int64_t stride, const float* f_bias, const float* lower,
                       float* state, int H, int d, int dv, const int32_t* cu, const int32_t* slots, const int32_t* pos,
                       int n_seg, bool f32, hipStream_t stream) {
  if (n_seg == 0) return true;
  if (f32)
    return launch_hgrn2_t<float>(out, (const float*)proj, stride, f_bias, lower, state, H, d, dv, cu, slots, pos, n_seg,
                                 stream);
  return launch_hgrn2_t<uint16_t>(out, (const uint16_t*)proj, stride, f_bias, lower, state, H, d, dv, cu, slots, pos,
                                  n_seg, stream);
}

}  // namespace nga
