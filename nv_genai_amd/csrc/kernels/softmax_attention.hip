// Softmax attention with head maps over row-major pages, and the projection-side kernel that
// feeds it.
//
//   headnorm_cache     per token row [q: nq heads of dk | k: nk heads of dk | v: nv heads of dv]:
//                      bias, RMS norm of every q head and every k head over its dk elements
//                      (weight per element, shared by the heads), query temperature
//                      1 + coef * ln(floor((p + 1) / every) + 1), q / k / v written back in
//                      place, k and v into the token's page slot
//   softmax_attention  one wave per (token row, head), prompt portions and single-token rows
//                      alike: keys by lane for q.k, value columns by lane for w.V, running
//                      maximum and sum per map (fp32); any sizes, bf16 and fp32
//   softmax_attention_mfma (bf16)  one workgroup per (64-row block of a sequence, head): MFMA q.k
//                      and p.V tiles over the pages the block can see, both maps in one wave
//   softmax_decode_mfma + softmax_decode_reduce (bf16)  single-token rows: the heads of a KV head
//                      are the tile columns, a row's pages are dealt to several workgroups
//
// Pages: K [blocks, G * maps, 64, dk], V [blocks, G, 64, dv] (T = bf16 or fp32). A head has
// `maps` score maps (1 or 2) that share its values: q head (h, m) is column block h * maps + m,
// its keys are k head (h / (H / G)) * maps + m. Two maps combine as a_0 - lam * a_1
// (differential attention). Optional: unit RMS of the head output (eps inside the root) times
// out_scale, and a per-head sigmoid gate. Visible keys of the query at position i: j <= i, and
// i - j < window when window > 0. v_row: elements between two value rows of a page; v_row = dk with
// vc = kc reads the values out of the first dv elements of the key rows (one map: a latent that is
// key and value, followed by key-only columns).
#include <cstdlib>

#include "common.h"
#include "kernels.h"

namespace nga {

namespace {

constexpr int BS = 64;   // tokens per page

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

// q . k over dk elements, q in LDS (fp32), k a page row; 16-byte loads when vec
__device__ __forceinline__ float dot_row(const float* qs, const uint16_t* kr, int dk, bool vec) {
  float s = 0.f;
  if (vec) {
    for (int d = 0; d < dk; d += 8) {
      const u16x8 k8 = load8(kr + d);
#pragma unroll
      for (int j = 0; j < 8; ++j) s += qs[d + j] * bf2f(k8[j]);
    }
  } else {
    for (int d = 0; d < dk; ++d) s += qs[d] * bf2f(kr[d]);
  }
  return s;
}
__device__ __forceinline__ float dot_row(const float* qs, const float* kr, int dk, bool vec) {
  float s = 0.f;
  if (vec) {
    for (int d = 0; d < dk; d += 4) {
      const float4 k4 = *reinterpret_cast<const float4*>(kr + d);
      s += qs[d] * k4.x + qs[d + 1] * k4.y + qs[d + 2] * k4.z + qs[d + 3] * k4.w;
    }
  } else {
    for (int d = 0; d < dk; ++d) s += qs[d] * kr[d];
  }
  return s;
}

template <typename T>
__global__ void __launch_bounds__(256) headnorm_cache_kernel(
    T* __restrict__ proj, int64_t stride, const int32_t* __restrict__ slots, T* __restrict__ kc, T* __restrict__ vc,
    int nq, int nk, int dk, int nv, int dv, float eps, const float* __restrict__ qw, const float* __restrict__ kw,
    const float* __restrict__ bias, const int32_t* __restrict__ pos, float coef, int every) {
  const int64_t row = blockIdx.x;
  T* pr = proj + row * stride;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float temp = 1.0f;
  if (coef != 0.f && nq > 0) {
    const int p = pos[row] < 0 ? 0 : pos[row];
    temp = 1.0f + coef * logf((float)((p + 1) / every + 1));
  }
  const int slot = slots[row];
  const int64_t page = slot >= 0 ? slot / BS : 0;
  const int off = slot >= 0 ? slot % BS : 0;
  for (int u = wave; u < nq + nk; u += 4) {
    const bool isq = u < nq;
    const float* w = isq ? qw : kw;
    const int base = u * dk;
    float r = 1.0f;
    if (w) {
      float ss = 0.f;
      for (int c = lane; c < dk; c += 64) {
        const float v = ldf(pr + base + c) + (bias ? bias[base + c] : 0.f);
        ss += v * v;
      }
      ss = wave_sum(ss);
      r = 1.0f / sqrtf(ss / (float)dk + eps);
    }
    T* kdst = (!isq && slot >= 0) ? kc + ((page * nk + (u - nq)) * BS + off) * (int64_t)dk : nullptr;
    for (int c = lane; c < dk; c += 64) {
      float v = ldf(pr + base + c) + (bias ? bias[base + c] : 0.f);
      if (w) v = v * r * w[c];
      if (isq) v *= temp;
      stf(pr + base + c, v);
      if (kdst) stf(kdst + c, v);
    }
  }
  const int vb = (nq + nk) * dk;
  for (int c = threadIdx.x; c < nv * dv; c += blockDim.x) {
    const float v = ldf(pr + vb + c) + (bias ? bias[vb + c] : 0.f);
    stf(pr + vb + c, v);
    if (slot >= 0) {
      const int hh = c / dv, d = c - hh * dv;
      stf(vc + ((page * nv + hh) * BS + off) * (int64_t)dv + d, v);
    }
  }
}

// One wave per (token row, head). q: row stride q_stride, head (h, m) at (h * maps + m) * dk.
// gate: row stride g_stride, one pre-sigmoid value per head (nullptr: no gate). out [T, H * dv].
template <typename T>
__global__ void __launch_bounds__(64) softmax_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ gate, int64_t g_stride,
    const T* __restrict__ kc, const T* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int H, int G, int dk, int dv, float scale,
    int window, int maps, float lam, float unit_eps, float out_scale, int v_row, float softcap) {
  extern __shared__ float smem[];
  float* qs = smem;                 // [maps * dk]
  float* ws = smem + maps * dk;     // [64]
  const int64_t row = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int i = pos[row];
  T* orow = out + row * (int64_t)H * dv + (int64_t)h * dv;
  if (i < 0) {   // padding row
    for (int d = lane; d < dv; d += 64) stf(orow + d, 0.f);
    return;
  }
  const int seq = tok_seq[row];
  const int g = h / (H / G);
  const int32_t* bt = block_tables + (int64_t)seq * max_blocks;
  for (int d = lane; d < maps * dk; d += 64) qs[d] = ldf(q + row * q_stride + (int64_t)h * maps * dk + d);
  constexpr int MAXV = 16;   // dv <= 1024
  float res[MAXV], acc[MAXV];
#pragma unroll
  for (int u = 0; u < MAXV; ++u) res[u] = 0.f;
  const int lo = window > 0 && i - window + 1 > 0 ? i - window + 1 : 0;
  const int p_lo = lo / BS, p_hi = i / BS;
  const bool vec = (dk % (16 / (int)sizeof(T))) == 0;
  __syncthreads();
  for (int m = 0; m < maps; ++m) {
    const int kh = g * maps + m;
    float mx = -INFINITY, l = 0.f;
#pragma unroll
    for (int u = 0; u < MAXV; ++u) acc[u] = 0.f;
    for (int p = p_lo; p <= p_hi; ++p) {
      const int j = p * BS + lane;
      const bool vis = j >= lo && j <= i;
      const int64_t page = bt[p];
      float s = -INFINITY;
      if (vis) {
        s = dot_row(qs + m * dk, kc + ((page * G * maps + kh) * BS + lane) * (int64_t)dk, dk, vec) * scale;
        if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      }
      const float nmx = fmaxf(mx, wave_max(s));   // every visited page holds a visible key
      const float corr = expf(mx - nmx);          // 0 on the first page (mx = -inf)
      const float w = vis ? expf(s - nmx) : 0.f;
      l = l * corr + wave_sum(w);
      mx = nmx;
      ws[lane] = w;
      __syncthreads();
      const unsigned long long any = __ballot(vis);
      const int j0 = __builtin_ctzll(any), j1 = 63 - __builtin_clzll(any);
      const T* vp = vc + ((page * G + g) * BS) * (int64_t)v_row;
#pragma unroll
      for (int u = 0; u < MAXV; ++u) {
        const int d = lane + u * 64;
        if (d < dv) {
          float a = acc[u] * corr;
          for (int jj = j0; jj <= j1; ++jj) a += ws[jj] * ldf(vp + (int64_t)jj * v_row + d);
          acc[u] = a;
        }
      }
      __syncthreads();
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int u = 0; u < MAXV; ++u) res[u] = m == 0 ? acc[u] * inv : res[u] - lam * (acc[u] * inv);
  }
  float r = 1.0f;
  if (unit_eps >= 0.f) {
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < MAXV; ++u)
      if (lane + u * 64 < dv) ss += res[u] * res[u];
    ss = wave_sum(ss);
    r = out_scale / sqrtf(ss / (float)dv + unit_eps);
  }
  if (gate) r *= sigmoidf_(ldf(gate + row * g_stride + h));
#pragma unroll
  for (int u = 0; u < MAXV; ++u) {
    const int d = lane + u * 64;
    if (d < dv) stf(orow + d, res[u] * r);
  }
}

// ---------------------------------------------------------------------------------------------
// MFMA form for prompt portions (bf16). Workgroup = 4 waves = 64 query rows of one sequence and
// one head; each wave owns 16 rows (the 16 columns of its mfma_f32_16x16x32_bf16 tiles) and runs
// all maps of the head, so a V page is staged once for both maps. Per 64-key page the workgroup
// stages K [maps][64][DK] in LDS (16-B chunks XOR-swizzled by row) and V transposed, V^T [DV][64]:
// a thread loads 4 keys x 8 value columns with 16-B loads, transposes them in registers and
// writes 8 rows x 4 keys with 8-byte stores. Every wave computes S^T = K . Q^T with the key rows
// permuted so that lane (query, h) ends up holding keys 32g + 8h .. + 7 of the page in its
// accumulators - exactly the B operand of O^T += V^T . P^T, so the weights never move between
// lanes. The softmax runs per query column in the exp2 domain: the running maximum and sum are
// reduced over the lane's 16 scores and the 4 lanes of its column; accumulators are rescaled
// when the maximum moves. Pages visited: those the block's windows cover.
// Soft cap of a score in the exp2 domain on the hardware exp2 and reciprocal:
// cap_log2 * tanh(x) with x = dot * scale / cap, as cap_log2 - 2 cap_log2 / (1 + 2^(k dot)),
// k = 2 log2(e) * scale / cap (five vector operations per score)
__device__ __forceinline__ float capped_score(float dot, float k, float cap_log2, float m2cap) {
  return m2cap * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(k * dot)) + cap_log2;
}

__device__ __forceinline__ int sm_row_swz(int row) { return (row & 3) | (((row >> 3) & 3) << 2); }

struct SmMfmaParams {
  uint16_t* out;             // [T, H * DV]
  const uint16_t* q;         // row stride q_stride, head (h, m) at (h * MAPS + m) * DK
  const uint16_t* gate;      // row stride g_stride, one value per head (nullptr: none)
  const uint16_t* kc;
  const uint16_t* vc;
  const int32_t* block_tables;
  const int32_t* cu_q;       // [B + 1] token rows of each sequence in this launch
  const int32_t* ctx_lens;   // [B] keys of each sequence after this step (its rows are the last ones)
  int64_t q_stride, g_stride;
  int max_blocks, H, G, window;
  float scale_log2, lam, unit_eps, out_scale;
  float cap_log2;            // soft cap of the scores times log2 e (0: none)
  int v_row;                 // elements between value rows of a page (DV, or DK when the values lie in the key rows)
};

// WPE: waves per SIMD the register allocation aims at. Large tiles (maps x DK + DV >= 192) are
// compiled for two: with the whole register file the scheduler keeps a tile's LDS reads in flight
// ahead of the MFMAs instead of reading fragment by fragment (2x faster at 128-wide heads, measured).
// SHARE (MAPS = 2): the wave's two score maps are two *heads* (2 hq, 2 hq + 1) of one KV head that
// read the same K tile - every K fragment is read from LDS once for both heads' MFMAs, as the V^T
// fragments are - and their outputs are written separately. With many heads over one page
// (multi-query attention over a latent) this halves the staging and the LDS reads per flop.
template <int DK, int DV, int MAPS, int WPE, bool SHARE = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
softmax_attention_mfma_kernel(const SmMfmaParams P) {
  static_assert(!SHARE || MAPS == 2, "two heads per wave");
  constexpr int KM = SHARE ? 1 : MAPS;     // K tiles staged per page
  constexpr int KT = 64;
  constexpr int NCH_K = DK / 8;
  constexpr int DS = DK / 32;
  constexpr int DT = DV / 16;
  constexpr int PER_K = DK / 32;           // 16-B chunks per thread per K page
  constexpr int VBLK = (2 * DV + 255) / 256;   // (4 keys x 8 columns) blocks per thread per V page
  // the XOR must stay inside an aligned group of chunks that the row holds whole: the largest
  // power of two dividing the chunk count (96-, 192-, 320-wide keys: 4, 8, 8 chunks)
  constexpr int P2 = NCH_K & -NCH_K;
  constexpr int SWS = P2 >= 16 ? 0 : P2 == 8 ? 1 : 2;
  extern __shared__ __attribute__((aligned(16))) uint16_t sm_lds[];
  uint16_t* k_s = sm_lds;                       // [KM][KT * DK]
  uint16_t* v_s = sm_lds + KM * KT * DK;        // [DV * KT]
  // Longest first: the row block is the slowest grid index and counts down, so the blocks that
  // see the most pages are dispatched first for every head and sequence, and the short ones fill
  // the gaps at the end (with the row block as the fastest index the second half of the grid
  // started its longest blocks late: the CUs were busy 56 % of a causal 8 x 2048-token launch).
  const int tile = gridDim.z - 1 - blockIdx.z, hq = blockIdx.x, b = blockIdx.y;
  const int q0 = P.cu_q[b], qlen = P.cu_q[b + 1] - q0;
  if (tile * 64 >= qlen) return;
  const int ctx = P.ctx_lens[b];
  const int g = (SHARE ? 2 * hq : hq) / (P.H / P.G);
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, h = lane >> 4;
  const int W = P.window;

  int r = tile * 64 + w * 16 + col;
  const bool row_ok = r < qlen;
  if (!row_ok) r = qlen - 1;
  const int qpos = ctx - qlen + r;
  bf16x8 qf[MAPS][DS];
  {
    const uint16_t* qp = P.q + (int64_t)(q0 + r) * P.q_stride + (int64_t)hq * MAPS * DK;
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
      for (int s2 = 0; s2 < DS; ++s2) qf[m][s2] = as_bf16x8(load8(qp + m * DK + 32 * s2 + 8 * h));
  }
  const int qpos_lo = ctx - qlen + tile * 64;
  const int qpos_hi = ctx - qlen + min(qlen - 1, tile * 64 + 63);
  const int lo_min = W > 0 ? max(0, qpos_lo - W + 1) : 0;
  const int t_first = lo_min / KT, t_last = qpos_hi / KT;
  const float fW = W > 0 ? (float)W : 3.0e38f;
  // positions of this wave's first and last rows
  const int wq_lo = ctx - qlen + min(qlen - 1, tile * 64 + w * 16);
  const int wq_hi = ctx - qlen + min(qlen - 1, tile * 64 + w * 16 + 15);

  f32x4 o[MAPS][DT];
  float mrun[MAPS], lrun[MAPS];
#pragma unroll
  for (int m = 0; m < MAPS; ++m) {
    mrun[m] = -INFINITY;
    lrun[m] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[m][dt] = (f32x4)(0.f);
  }

  // Registers for one page in flight: with few enough of them the next page is requested before
  // the current one is processed, so its latency hides behind the MFMA work.
  constexpr bool PREFETCH = (KM * PER_K + 4 * VBLK) * 4 <= 48;
  u16x8 kreg[KM][PER_K], vreg[VBLK][4];
  // the page number of the next fetch is looked up one iteration ahead, so that the page loads do
  // not wait for the table
  const int32_t* btp = P.block_tables + (int64_t)b * P.max_blocks;
  int blk_next = btp[t_first];
  auto fetch = [&](int64_t blk) {
    const uint16_t* kp = P.kc + (blk * P.G + g) * (int64_t)(KM * KT * DK);
    const uint16_t* vp = P.vc + (blk * P.G + g) * (int64_t)KT * P.v_row;
#pragma unroll
    for (int m = 0; m < KM; ++m)
#pragma unroll
      for (int i = 0; i < PER_K; ++i) kreg[m][i] = load8(kp + m * KT * DK + (int64_t)(tid + 256 * i) * 8);
#pragma unroll
    for (int i = 0; i < VBLK; ++i) {
      const int c = tid + 256 * i;            // block: keys 4 * (c & 15) .. + 3, columns 8 * (c >> 4) .. + 7
      if (c < 2 * DV) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) vreg[i][kk] = load8(vp + (int64_t)(4 * (c & 15) + kk) * P.v_row + 8 * (c >> 4));
      }
    }
  };
  fetch(blk_next);
  if (t_first < t_last) blk_next = btp[t_first + 1];
  for (int t = t_first; t <= t_last; ++t) {
    __syncthreads();   // the previous page's reads are done
#pragma unroll
    for (int m = 0; m < KM; ++m)
#pragma unroll
      for (int i = 0; i < PER_K; ++i) {
        const int c = tid + 256 * i;
        const int row = c / NCH_K, ch = c % NCH_K;
        const int sw = sm_row_swz(row) >> SWS;
        *reinterpret_cast<u16x8*>(&k_s[m * KT * DK + row * DK + ((ch ^ sw) * 8)]) = kreg[m][i];
      }
#pragma unroll
    for (int i = 0; i < VBLK; ++i) {
      const int c = tid + 256 * i;
      if (c < 2 * DV) {
        const int kb = c & 15, dc = c >> 4;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int row = 8 * dc + e;
          u16x4 tv;
          tv[0] = vreg[i][0][e];
          tv[1] = vreg[i][1][e];
          tv[2] = vreg[i][2][e];
          tv[3] = vreg[i][3][e];
          *reinterpret_cast<u16x4*>(&v_s[row * KT + (((kb >> 1) ^ ((row >> 1) & 7)) * 8) + 4 * (kb & 1)]) = tv;
        }
      }
    }
    __syncthreads();
    if (PREFETCH && t < t_last) {
      fetch(blk_next);
      if (t + 1 < t_last) blk_next = btp[t + 2];
    }

    const int kbase = t * KT;
    const float fd = (float)(qpos - kbase - 8 * h);
    const bool need_mask = kbase + KT - 1 > wq_lo || (W > 0 && wq_hi - kbase >= W);
    const bool capped = P.cap_log2 > 0.f;
    const float cap_k = capped ? 2.8853900817779268f * P.scale_log2 / P.cap_log2 : 0.f, cap_m2 = -2.0f * P.cap_log2;
    bf16x8 pf[MAPS][2];
    f32x4 sboth[SHARE ? MAPS : 1][4];
    if constexpr (SHARE) {   // both heads' scores from one read of every K fragment
#pragma unroll
      for (int tau = 0; tau < 4; ++tau) {
        const int row = 32 * (tau >> 1) + 8 * (col >> 2) + 4 * (tau & 1) + (col & 3);
        const int sw = sm_row_swz(row) >> SWS;
#pragma unroll
        for (int m = 0; m < MAPS; ++m) sboth[m][tau] = (f32x4)(0.f);
#pragma unroll
        for (int s2 = 0; s2 < DS; ++s2) {
          const int ch = 4 * s2 + h;
          const bf16x8 a = as_bf16x8(*reinterpret_cast<const u16x8*>(&k_s[row * DK + ((ch ^ sw) * 8)]));
#pragma unroll
          for (int m = 0; m < MAPS; ++m) sboth[m][tau] = mfma16(a, qf[m][s2], sboth[m][tau]);
        }
      }
    }
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      f32x4 sacc[4];
#pragma unroll
      for (int tau = 0; tau < 4; ++tau) {
        if constexpr (SHARE) {
          sacc[tau] = sboth[m][tau];
        } else {
          const int row = 32 * (tau >> 1) + 8 * (col >> 2) + 4 * (tau & 1) + (col & 3);
          const int sw = sm_row_swz(row) >> SWS;
          sacc[tau] = (f32x4)(0.f);
#pragma unroll
          for (int s2 = 0; s2 < DS; ++s2) {
            const int ch = 4 * s2 + h;
            const bf16x8 a = as_bf16x8(*reinterpret_cast<const u16x8*>(&k_s[m * KT * DK + row * DK + ((ch ^ sw) * 8)]));
            sacc[tau] = mfma16(a, qf[m][s2], sacc[tau]);
          }
        }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int tau = 0; tau < 4; ++tau)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          float sv = sacc[tau][rr] * P.scale_log2;
          if (capped) sv = capped_score(sacc[tau][rr], cap_k, P.cap_log2, cap_m2);
          if (need_mask) {
            const float d = fd - (float)(32 * (tau >> 1) + 4 * (tau & 1) + rr);
            sv = (d >= 0.f && d < fW) ? sv : -INFINITY;
          }
          sacc[tau][rr] = sv;
          mx = fmaxf(mx, sv);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mnew = fmaxf(mrun[m], mx);
      const float muse = mnew == -INFINITY ? 0.f : mnew;   // nothing visible yet: weights and factor 0
      const float corr = __builtin_amdgcn_exp2f(mrun[m] - muse);
      const bool moved = mnew != mrun[m];
      mrun[m] = mnew;
      float ls = 0.f;
#pragma unroll
      for (int tau = 0; tau < 4; ++tau)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const float pv = __builtin_amdgcn_exp2f(sacc[tau][rr] - muse);
          ls += pv;
          pf[m][tau >> 1][4 * (tau & 1) + rr] = (__bf16)pv;
        }
      ls += __shfl_xor(ls, 16, 64);
      ls += __shfl_xor(ls, 32, 64);
      lrun[m] = lrun[m] * corr + ls;
      if (__ballot(moved)) {   // no maximum of this wave's rows moved: the accumulators stay as they are
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[m][dt] *= corr;
      }
    }
#pragma unroll
    for (int gg = 0; gg < 2; ++gg) {
      const int ch = 4 * gg + h;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const int row = 16 * dt + col;
        const bf16x8 a = as_bf16x8(*reinterpret_cast<const u16x8*>(&v_s[row * KT + ((ch ^ ((row >> 1) & 7)) * 8)]));
#pragma unroll
        for (int m = 0; m < MAPS; ++m) o[m][dt] = mfma16(a, pf[m][gg], o[m][dt]);
      }
    }
    if (!PREFETCH && t < t_last) {
      fetch(blk_next);
      if (t + 1 < t_last) blk_next = btp[t + 2];
    }
  }
  // lane (query col, h) holds value columns 16 dt + 4 h + rr of its query
  float inv[MAPS];
#pragma unroll
  for (int m = 0; m < MAPS; ++m) inv[m] = 1.0f / lrun[m];
  if constexpr (SHARE) {   // two heads: each normalised, scaled, gated and written on its own
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      float s2 = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const float v = o[m][dt][rr] * inv[m];
          o[m][dt][rr] = v;
          s2 += v * v;
        }
      float rs = 1.0f;
      if (P.unit_eps >= 0.f) {
        s2 += __shfl_xor(s2, 16, 64);
        s2 += __shfl_xor(s2, 32, 64);
        rs = P.out_scale / sqrtf(s2 / (float)DV + P.unit_eps);
      }
      if (row_ok) {
        const int head = 2 * hq + m;
        if (P.gate) rs *= sigmoidf_(bf2f(P.gate[(int64_t)(q0 + r) * P.g_stride + head]));
        uint16_t* op = P.out + (int64_t)(q0 + r) * P.H * DV + (int64_t)head * DV;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          u16x4 ov;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) ov[rr] = f2bf(o[m][dt][rr] * rs);
          *reinterpret_cast<u16x4*>(op + 16 * dt + 4 * h) = ov;
        }
      }
    }
    return;
  }
  float ss = 0.f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      float v = o[0][dt][rr] * inv[0];
      if (MAPS == 2) v -= P.lam * (o[MAPS - 1][dt][rr] * inv[MAPS - 1]);
      o[0][dt][rr] = v;
      ss += v * v;
    }
  float rs = 1.0f;
  if (P.unit_eps >= 0.f) {
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    rs = P.out_scale / sqrtf(ss / (float)DV + P.unit_eps);
  }
  if (!row_ok) return;
  if (P.gate) rs *= sigmoidf_(bf2f(P.gate[(int64_t)(q0 + r) * P.g_stride + hq]));
  uint16_t* op = P.out + (int64_t)(q0 + r) * P.H * DV + (int64_t)hq * DV;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    u16x4 ov;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) ov[rr] = f2bf(o[0][dt][rr] * rs);
    *reinterpret_cast<u16x4*>(op + 16 * dt + 4 * h) = ov;
  }
}

template <int DK, int DV, int MAPS>
void launch_sm_mfma_one(const SmMfmaParams& P, dim3 grid, hipStream_t stream) {
  constexpr size_t smem = (size_t)(MAPS * 64 * DK + DV * 64) * sizeof(uint16_t);
  constexpr int WPE = MAPS * DK + DV >= 192 ? 2 : (MAPS * DK + DV >= 128 ? 3 : 4);
  static bool attr_set = false;   // more than 64 KB of dynamic LDS needs the attribute once
  if (smem > 65536 && !attr_set) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&softmax_attention_mfma_kernel<DK, DV, MAPS, WPE>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    attr_set = true;
  }
  softmax_attention_mfma_kernel<DK, DV, MAPS, WPE><<<grid, 256, smem, stream>>>(P);
}

template <int DK, int MAPS>
bool launch_sm_mfma_dv(const SmMfmaParams& P, int dv, dim3 grid, hipStream_t stream) {
  switch (dv) {
    case 32: launch_sm_mfma_one<DK, 32, MAPS>(P, grid, stream); return true;
    case 64: launch_sm_mfma_one<DK, 64, MAPS>(P, grid, stream); return true;
    case 128: launch_sm_mfma_one<DK, 128, MAPS>(P, grid, stream); return true;
    case 256:
      if (MAPS == 1) {
        launch_sm_mfma_one<DK, 256, 1>(P, grid, stream);
        return true;
      }
      return false;
    default: return false;
  }
}

// two heads of one KV head per wave over a shared K tile (one map per head)
template <int DK, int DV>
void launch_sm_mfma_shared(const SmMfmaParams& P, dim3 grid, hipStream_t stream) {
  constexpr size_t smem = (size_t)(64 * DK + DV * 64) * sizeof(uint16_t);
  static_assert(smem <= 65536, "dynamic LDS without the attribute");
  grid.x = (unsigned)(P.H / 2);
  softmax_attention_mfma_kernel<DK, DV, 2, 2, true><<<grid, 256, smem, stream>>>(P);
}

// key sizes of a latent plus a rotated part (one map): one value size each. SHARED: an even number
// of heads per KV head runs two heads per wave (both heads' accumulators fit two waves per SIMD;
// at 320-wide keys they do not, and one wave per SIMD measured twice as slow as one head per wave).
template <int DK, int DV, bool SHARED>
bool launch_sm_mfma_pair(const SmMfmaParams& P, int dv, dim3 grid, hipStream_t stream) {
  if (dv != DV) return false;
  if constexpr (SHARED) {
    if (kernel_form(KF_SM_SHARE_HEADS) != 0 && (P.H / P.G) % 2 == 0) {
      launch_sm_mfma_shared<DK, DV>(P, grid, stream);
      return true;
    }
  }
  launch_sm_mfma_one<DK, DV, 1>(P, grid, stream);
  return true;
}

template <int MAPS>
bool launch_sm_mfma_dk(const SmMfmaParams& P, int dk, int dv, dim3 grid, hipStream_t stream) {
  if (MAPS == 1) {
    if (dk == 96) return launch_sm_mfma_pair<96, 64, true>(P, dv, grid, stream);
    if (dk == 192) return launch_sm_mfma_pair<192, 128, true>(P, dv, grid, stream);
    if (dk == 320) return launch_sm_mfma_pair<320, 256, false>(P, dv, grid, stream);
  }
  switch (dk) {
    case 32: return launch_sm_mfma_dv<32, MAPS>(P, dv, grid, stream);
    case 64: return launch_sm_mfma_dv<64, MAPS>(P, dv, grid, stream);
    case 128: return launch_sm_mfma_dv<128, MAPS>(P, dv, grid, stream);
    case 256: return MAPS == 1 ? launch_sm_mfma_dv<256, 1>(P, dv, grid, stream) : false;
    default: return false;
  }
}

// ---------------------------------------------------------------------------------------------
// MFMA form for single-token rows (bf16): the columns of the 16-wide tiles are the heads that
// share one KV head (16 per workgroup), so a page is read once for the whole group (and once for
// both maps of a head: they share V). Workgroup = 4 waves = (part, KV head, token row); the row's visible pages
// are dealt round-robin to the 4 * parts waves of the row. K fragments go from the page straight
// into the MFMA A operand; V is transposed through a wave-private LDS tile (V^T [DV][64], as in
// the prompt kernel). Every wave keeps its own running (max, sum, accumulator) per head and map;
// the four waves merge theirs through LDS into one partial per workgroup, and
// softmax_decode_reduce merges the partials of a (row, head) in a fixed order, combines the maps,
// normalises, gates and writes bf16.
//
// ws: fp32 [T, H, MAPS, parts, DV + 4]  (accumulator, then max (log2 domain), sum, 2 unused)
template <int DK, int DV, int MAPS>
__device__ __forceinline__ void softmax_decode_mfma_body(
    float* __restrict__ ws, const uint16_t* __restrict__ q, int64_t q_stride, const uint16_t* __restrict__ kc,
    const uint16_t* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int H, int G, float scale_log2, float cap_log2, int window,
    int v_row) {
  constexpr int KT = 64;
  constexpr int DS = DK / 32;
  constexpr int DT = DV / 16;
  constexpr int VBLK = DV / 32;   // (4 keys x 8 columns) blocks per lane per page
  extern __shared__ __attribute__((aligned(16))) uint16_t sm_lds[];
  const int grp = H / G;
  const int n_chunk = (grp + 15) / 16;   // more than 16 heads per KV head: 16 per workgroup
  const int part = blockIdx.x, parts = gridDim.x, g = blockIdx.y / n_chunk, c0 = (blockIdx.y % n_chunk) * 16;
  const int64_t row = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  uint16_t* v_s = sm_lds + w * (DV * KT);
  const int col = lane & 15, h = lane >> 4;
  const int head = g * grp + (c0 + col < grp ? c0 + col : grp - 1);
  const int i = pos[row];
  const int lo = window > 0 && i - window + 1 > 0 ? i - window + 1 : 0;
  const int p_lo = lo / KT, p_hi = i / KT;           // i < 0: no pages
  const int n_pages = i < 0 ? 0 : p_hi - p_lo + 1;
  const int stride = 4 * parts;
  const int n_it = (n_pages + stride - 1) / stride;  // the same for all four waves (barriers inside)
  const int32_t* bt = block_tables + (int64_t)tok_seq[row] * max_blocks;

  bf16x8 qf[MAPS][DS];
  {
    const uint16_t* qp = q + row * q_stride + (int64_t)head * MAPS * DK;
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
      for (int s2 = 0; s2 < DS; ++s2) qf[m][s2] = as_bf16x8(load8(qp + m * DK + 32 * s2 + 8 * h));
  }
  f32x4 o[MAPS][DT];
  float mrun[MAPS], lrun[MAPS];
#pragma unroll
  for (int m = 0; m < MAPS; ++m) {
    mrun[m] = -INFINITY;
    lrun[m] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[m][dt] = (f32x4)(0.f);
  }

  for (int it = 0; it < n_it; ++it) {
    const int pg = p_lo + it * stride + part * 4 + w;
    const bool have = pg <= p_hi;
    const int64_t blk = have ? bt[pg] : 0;
    const uint16_t* kp = kc + (blk * G + g) * (int64_t)(MAPS * KT * DK);
    const uint16_t* vp = vc + (blk * G + g) * (int64_t)KT * v_row;
    __syncthreads();   // the previous page's reads of this wave's tile are done
    if (have) {
      // all of the page's V loads in flight together, then the transposed stores
      u16x8 vreg[VBLK][4];
#pragma unroll
      for (int bi = 0; bi < VBLK; ++bi) {
        const int c = lane + 64 * bi;            // block: keys 4 * (c & 15) .. + 3, columns 8 * (c >> 4) .. + 7
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) vreg[bi][kk] = load8(vp + (int64_t)(4 * (c & 15) + kk) * v_row + 8 * (c >> 4));
      }
#pragma unroll
      for (int bi = 0; bi < VBLK; ++bi) {
        const int c = lane + 64 * bi;
        const int kb = c & 15, dc = c >> 4;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int r = 8 * dc + e;
          u16x4 tv;
          tv[0] = vreg[bi][0][e];
          tv[1] = vreg[bi][1][e];
          tv[2] = vreg[bi][2][e];
          tv[3] = vreg[bi][3][e];
          *reinterpret_cast<u16x4*>(&v_s[r * KT + (((kb >> 1) ^ ((r >> 1) & 7)) * 8) + 4 * (kb & 1)]) = tv;
        }
      }
    }
    __syncthreads();
    if (!have) continue;
    const int kbase = pg * KT;
    const bool need_mask = kbase < lo || kbase + KT - 1 > i;
    const bool capped = cap_log2 > 0.f;
    const float cap_k = capped ? 2.8853900817779268f * scale_log2 / cap_log2 : 0.f, cap_m2 = -2.0f * cap_log2;
    bf16x8 pf[MAPS][2];
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      // the map's K fragments of the whole page in flight together (one round trip), then the MFMAs
      u16x8 kf[4][DS];
#pragma unroll
      for (int tau = 0; tau < 4; ++tau) {
        const int kr = 32 * (tau >> 1) + 8 * (col >> 2) + 4 * (tau & 1) + (col & 3);
#pragma unroll
        for (int s2 = 0; s2 < DS; ++s2) kf[tau][s2] = load8(kp + m * KT * DK + kr * DK + 32 * s2 + 8 * h);
      }
      f32x4 sacc[4];
#pragma unroll
      for (int tau = 0; tau < 4; ++tau) {
        sacc[tau] = (f32x4)(0.f);
#pragma unroll
        for (int s2 = 0; s2 < DS; ++s2) sacc[tau] = mfma16(as_bf16x8(kf[tau][s2]), qf[m][s2], sacc[tau]);
      }
      float mx = -INFINITY;
#pragma unroll
      for (int tau = 0; tau < 4; ++tau)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          float sv = sacc[tau][rr] * scale_log2;
          if (capped) sv = capped_score(sacc[tau][rr], cap_k, cap_log2, cap_m2);
          if (need_mask) {
            const int j = kbase + 32 * (tau >> 1) + 8 * h + 4 * (tau & 1) + rr;
            sv = (j >= lo && j <= i) ? sv : -INFINITY;
          }
          sacc[tau][rr] = sv;
          mx = fmaxf(mx, sv);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mnew = fmaxf(mrun[m], mx);     // every visited page holds a visible key
      const float corr = __builtin_amdgcn_exp2f(mrun[m] - mnew);
      const bool moved = mnew != mrun[m];
      mrun[m] = mnew;
      float ls = 0.f;
#pragma unroll
      for (int tau = 0; tau < 4; ++tau)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const float pv = __builtin_amdgcn_exp2f(sacc[tau][rr] - mnew);
          ls += pv;
          pf[m][tau >> 1][4 * (tau & 1) + rr] = (__bf16)pv;
        }
      ls += __shfl_xor(ls, 16, 64);
      ls += __shfl_xor(ls, 32, 64);
      lrun[m] = lrun[m] * corr + ls;
      if (__ballot(moved)) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[m][dt] *= corr;
      }
    }
#pragma unroll
    for (int gg = 0; gg < 2; ++gg) {
      const int ch = 4 * gg + h;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const int r = 16 * dt + col;
        const bf16x8 a = as_bf16x8(*reinterpret_cast<const u16x8*>(&v_s[r * KT + ((ch ^ ((r >> 1) & 7)) * 8)]));
#pragma unroll
        for (int m = 0; m < MAPS; ++m) o[m][dt] = mfma16(a, pf[m][gg], o[m][dt]);
      }
    }
  }
  // merge the four waves' (max, sum, accumulator) through LDS (the V^T tiles are free now): the
  // workgroup leaves one partial per head and map
  __syncthreads();
  float* ml_s = reinterpret_cast<float*>(sm_lds);          // [4][MAPS][2][16]
  float* o_s = ml_s + 4 * MAPS * 2 * 16;                   // [MAPS][16][DV]
  if (h == 0) {
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      ml_s[((w * MAPS + m) * 2 + 0) * 16 + col] = mrun[m];
      ml_s[((w * MAPS + m) * 2 + 1) * 16 + col] = lrun[m];
    }
  }
  __syncthreads();
  float fac[MAPS], Mx[MAPS], Lx[MAPS];
#pragma unroll
  for (int m = 0; m < MAPS; ++m) {
    float M = -INFINITY;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) M = fmaxf(M, ml_s[((ww * MAPS + m) * 2 + 0) * 16 + col]);
    float L = 0.f;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) {
      const float mw = ml_s[((ww * MAPS + m) * 2 + 0) * 16 + col];
      if (mw != -INFINITY) L += ml_s[((ww * MAPS + m) * 2 + 1) * 16 + col] * __builtin_amdgcn_exp2f(mw - M);
    }
    fac[m] = mrun[m] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mrun[m] - M);
    Mx[m] = M;
    Lx[m] = L;
  }
#pragma unroll
  for (int ww = 0; ww < 4; ++ww) {
    if (w == ww) {
#pragma unroll
      for (int m = 0; m < MAPS; ++m)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          f32x4* dst = reinterpret_cast<f32x4*>(o_s + (m * 16 + col) * DV + 16 * dt + 4 * h);
          *dst = ww == 0 ? o[m][dt] * fac[m] : *dst + o[m][dt] * fac[m];
        }
    }
    __syncthreads();
  }
  // 16 heads x DV columns per map, written by all four waves
  const int stride_ws = parts;
  for (int e = tid; e < MAPS * 16 * (DV / 4); e += 256) {
    const int m = e / (16 * (DV / 4)), rem = e % (16 * (DV / 4)), cc = rem / (DV / 4), d4 = rem % (DV / 4);
    if (c0 + cc < grp) {
      float* wp = ws + ((((int64_t)row * H + g * grp + c0 + cc) * MAPS + m) * stride_ws + part) * (DV + 4);
      *reinterpret_cast<f32x4*>(wp + 4 * d4) = *reinterpret_cast<const f32x4*>(o_s + (m * 16 + cc) * DV + 4 * d4);
    }
  }
  if (w == 0 && h == 0 && c0 + col < grp) {
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      float* wp = ws + ((((int64_t)row * H + g * grp + c0 + col) * MAPS + m) * stride_ws + part) * (DV + 4);
      wp[DV] = Mx[m];
      wp[DV + 1] = Lx[m];
    }
  }
}

// Two entry points of the same body: two maps per head are compiled for two waves per SIMD (the
// scheduler then keeps a page's loads in flight ahead of the MFMAs: 0.091 -> 0.067 ms at 64 rows x
// 2048 keys); one map is faster with the default allocation (measured at 256-wide latents).
template <int DK, int DV, int MAPS>
__global__ void __launch_bounds__(256) softmax_decode_mfma_kernel(
    float* __restrict__ ws, const uint16_t* __restrict__ q, int64_t q_stride, const uint16_t* __restrict__ kc,
    const uint16_t* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int H, int G, float scale_log2, float cap_log2, int window,
    int v_row) {
  softmax_decode_mfma_body<DK, DV, MAPS>(ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, H, G, scale_log2, cap_log2,
                                         window, v_row);
}

template <int DK, int DV, int MAPS>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) softmax_decode_mfma_kernel_w2(
    float* __restrict__ ws, const uint16_t* __restrict__ q, int64_t q_stride, const uint16_t* __restrict__ kc,
    const uint16_t* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int H, int G, float scale_log2, float cap_log2, int window,
    int v_row) {
  softmax_decode_mfma_body<DK, DV, MAPS>(ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, H, G, scale_log2, cap_log2,
                                         window, v_row);
}

// one wave per (token row, head): merge the partials of each map, a_0 - lam * a_1, unit RMS, gate
__global__ void __launch_bounds__(64) softmax_decode_reduce_kernel(
    uint16_t* __restrict__ out, const float* __restrict__ ws, int slots, const uint16_t* __restrict__ gate,
    int64_t g_stride, int H, int dv, int maps, float lam, float unit_eps, float out_scale) {
  const int64_t row = blockIdx.x;
  const int head = blockIdx.y, lane = threadIdx.x;
  constexpr int MAXV = 4;   // dv <= 256
  float res[MAXV] = {0.f, 0.f, 0.f, 0.f};
  for (int m = 0; m < maps; ++m) {
    const float* wp = ws + (((int64_t)row * H + head) * maps + m) * slots * (int64_t)(dv + 4);
    float M = -INFINITY;
#pragma unroll 4
    for (int s = 0; s < slots; ++s) M = fmaxf(M, wp[(int64_t)s * (dv + 4) + dv]);
    float L = 0.f, acc[MAXV] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int s = 0; s < slots; ++s) {
      const float* sp = wp + (int64_t)s * (dv + 4);
      const float ms = sp[dv];
      if (ms == -INFINITY) continue;   // a wave that got no page
      const float f = __builtin_amdgcn_exp2f(ms - M);
      L += sp[dv + 1] * f;
#pragma unroll
      for (int u = 0; u < MAXV; ++u)
        if (lane + 64 * u < dv) acc[u] += sp[lane + 64 * u] * f;
    }
    const float inv = L > 0.f ? 1.0f / L : 0.f;   // padding row: zeros
#pragma unroll
    for (int u = 0; u < MAXV; ++u) res[u] = m == 0 ? acc[u] * inv : res[u] - lam * (acc[u] * inv);
  }
  float r = 1.0f;
  if (unit_eps >= 0.f) {
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < MAXV; ++u)
      if (lane + 64 * u < dv) ss += res[u] * res[u];
    ss = wave_sum(ss);
    r = out_scale / sqrtf(ss / (float)dv + unit_eps);
  }
  if (gate) r *= sigmoidf_(bf2f(gate[row * g_stride + head]));
#pragma unroll
  for (int u = 0; u < MAXV; ++u)
    if (lane + 64 * u < dv) out[(row * H + head) * (int64_t)dv + lane + 64 * u] = f2bf(res[u] * r);
}

template <int DK, int DV, int MAPS>
void launch_sm_decode_one(float* ws, const uint16_t* q, int64_t q_stride, const uint16_t* kc, const uint16_t* vc,
                          const int32_t* block_tables, int max_blocks, const int32_t* tok_seq, const int32_t* pos,
                          int H, int G, float scale_log2, float cap_log2, int window, int v_row, dim3 grid, hipStream_t stream) {
  constexpr size_t tiles = (size_t)4 * DV * 64 * sizeof(uint16_t);
  constexpr size_t merge = (size_t)(4 * MAPS * 2 * 16 + MAPS * 16 * DV) * sizeof(float);
  constexpr size_t smem = tiles > merge ? tiles : merge;
  static bool attr_set = false;
  if constexpr (MAPS == 2) {
    if (smem > 65536 && !attr_set) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&softmax_decode_mfma_kernel_w2<DK, DV, MAPS>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      attr_set = true;
    }
    softmax_decode_mfma_kernel_w2<DK, DV, MAPS><<<grid, 256, smem, stream>>>(ws, q, q_stride, kc, vc, block_tables,
                                                                            max_blocks, tok_seq, pos, H, G, scale_log2, cap_log2,
                                                                            window, v_row);
  } else {
    if (smem > 65536 && !attr_set) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&softmax_decode_mfma_kernel<DK, DV, MAPS>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      attr_set = true;
    }
    softmax_decode_mfma_kernel<DK, DV, MAPS><<<grid, 256, smem, stream>>>(ws, q, q_stride, kc, vc, block_tables,
                                                                         max_blocks, tok_seq, pos, H, G, scale_log2, cap_log2,
                                                                         window, v_row);
  }
}

#define NGA_SM_DEC_ARGS ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, H, G, scale_log2, cap_log2, window, v_row, grid, stream
template <int DK, int MAPS>
bool launch_sm_decode_dv(float* ws, const uint16_t* q, int64_t q_stride, const uint16_t* kc, const uint16_t* vc,
                         const int32_t* block_tables, int max_blocks, const int32_t* tok_seq, const int32_t* pos, int H,
                         int G, float scale_log2, float cap_log2, int window, int v_row, int dv, dim3 grid, hipStream_t stream) {
  switch (dv) {
    case 32: launch_sm_decode_one<DK, 32, MAPS>(NGA_SM_DEC_ARGS); return true;
    case 64: launch_sm_decode_one<DK, 64, MAPS>(NGA_SM_DEC_ARGS); return true;
    case 128: launch_sm_decode_one<DK, 128, MAPS>(NGA_SM_DEC_ARGS); return true;
    case 256:
      if (MAPS == 1) {
        launch_sm_decode_one<DK, 256, 1>(NGA_SM_DEC_ARGS);
        return true;
      }
      return false;
    default: return false;
  }
}

template <int MAPS>
bool launch_sm_decode_dk(float* ws, const uint16_t* q, int64_t q_stride, const uint16_t* kc, const uint16_t* vc,
                         const int32_t* block_tables, int max_blocks, const int32_t* tok_seq, const int32_t* pos, int H,
                         int G, float scale_log2, float cap_log2, int window, int v_row, int dk, int dv, dim3 grid, hipStream_t stream) {
#define NGA_SM_DEC_DV(DKV) launch_sm_decode_dv<DKV, MAPS>(ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, H, G, scale_log2, cap_log2, window, v_row, dv, grid, stream)
  if (MAPS == 1) {   // key sizes of a latent plus a rotated part: one value size each
    if (dk == 96 && dv == 64) { launch_sm_decode_one<96, 64, 1>(NGA_SM_DEC_ARGS); return true; }
    if (dk == 192 && dv == 128) { launch_sm_decode_one<192, 128, 1>(NGA_SM_DEC_ARGS); return true; }
    if (dk == 320 && dv == 256) { launch_sm_decode_one<320, 256, 1>(NGA_SM_DEC_ARGS); return true; }
  }
  switch (dk) {
    case 32: return NGA_SM_DEC_DV(32);
    case 64: return NGA_SM_DEC_DV(64);
    case 128: return NGA_SM_DEC_DV(128);
    case 256: return MAPS == 1 ? launch_sm_decode_dv<256, 1>(ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, H, G, scale_log2, cap_log2, window, v_row, dv, grid, stream) : false;
    default: return false;
  }
#undef NGA_SM_DEC_DV
}
#undef NGA_SM_DEC_ARGS

}  // namespace

// Parts (workgroups per row and KV head) of the single-token MFMA kernel: enough waves to fill
// the chip, never more than the pages a row can see. Fixed by sizes the host knows, so a
// captured step keeps its launch shape.
int softmax_decode_parts(int rows, int G, int max_ctx, int window) {
  const int64_t span = window > 0 && window < max_ctx ? window : max_ctx;
  const int pages = (int)(span / 64) + 2;
  const int by_pages = (pages + 3) / 4;
  const int target = 8192;   // waves to launch: 8 per SIMD on 256 CUs
  const int by_fill = (target + rows * G * 4 - 1) / (rows * G * 4);
  const int p = by_pages < by_fill ? by_pages : by_fill;
  return p < 1 ? 1 : (p > 32 ? 32 : p);
}

// ws: fp32 [T, H, maps, parts, dv + 4]
void launch_softmax_decode_mfma(uint16_t* out, float* ws, int parts, const uint16_t* q, int64_t q_stride,
                                const uint16_t* gate, int64_t g_stride, const uint16_t* kc, const uint16_t* vc,
                                const int32_t* block_tables, int max_blocks, const int32_t* tok_seq,
                                const int32_t* pos, int64_t T, int H, int G, int dk, int dv, float scale, int window,
                                int maps, float lam, float unit_eps, float out_scale, bool v_in_k, float softcap,
                                hipStream_t stream) {
  if (T == 0) return;
  const dim3 grid((unsigned)parts, (unsigned)(G * ((H / G + 15) / 16)), (unsigned)T);
  const float scale_log2 = scale * 1.4426950408889634f;
  const float cap_log2 = softcap > 0.f ? softcap * 1.4426950408889634f : 0.f;
  const int v_row = v_in_k ? dk : dv;
  const bool ok = maps == 2 ? launch_sm_decode_dk<2>(ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, H, G,
                                                     scale_log2, cap_log2, window, v_row, dk, dv, grid, stream)
                            : launch_sm_decode_dk<1>(ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, H, G,
                                                     scale_log2, cap_log2, window, v_row, dk, dv, grid, stream);
  if (!ok) abort();   // the caller checks softmax_attention_mfma_supported
  softmax_decode_reduce_kernel<<<dim3((unsigned)T, (unsigned)H), 64, 0, stream>>>(out, ws, parts, gate, g_stride, H,
                                                                                   dv, maps, lam, unit_eps, out_scale);
}

// Head sizes of the MFMA forms: dk, dv in {32, 64, 128} (one map: also 256, and the pairs
// (96, 64), (192, 128), (320, 256) of a latent with a rotated key part).
bool softmax_attention_mfma_supported(int dk, int dv, int group, int maps) {
  auto ok = [&](int d) { return d == 32 || d == 64 || d == 128 || (maps == 1 && d == 256); };
  if (maps == 1 && group >= 1 && ((dk == 96 && dv == 64) || (dk == 192 && dv == 128) || (dk == 320 && dv == 256)))
    return true;
  return (maps == 1 || maps == 2) && ok(dk) && ok(dv) && group >= 1;
}

// prompt portions: sequence b owns rows [cu_q[b], cu_q[b + 1]) of q / gate / out, the last ones of
// its ctx_lens[b] keys. q rows must be 16-byte aligned (checked by the caller).
void launch_softmax_attention_mfma(uint16_t* out, const uint16_t* q, int64_t q_stride, const uint16_t* gate,
                                   int64_t g_stride, const uint16_t* kc, const uint16_t* vc,
                                   const int32_t* block_tables, int max_blocks, const int32_t* cu_q,
                                   const int32_t* ctx_lens, int B, int max_q_len, int H, int G, int dk, int dv,
                                   float scale, int window, int maps, float lam, float unit_eps, float out_scale,
                                   bool v_in_k, float softcap, hipStream_t stream) {
  if (B == 0 || max_q_len == 0) return;
  SmMfmaParams P{out, q, gate, kc, vc, block_tables, cu_q, ctx_lens, q_stride, g_stride, max_blocks, H, G, window,
                 scale * 1.4426950408889634f, lam, unit_eps, out_scale,
                 softcap > 0.f ? softcap * 1.4426950408889634f : 0.f, v_in_k ? dk : dv};
  const dim3 grid((unsigned)H, (unsigned)B, (unsigned)((max_q_len + 63) / 64));   // (head, sequence, row block)
  const bool ok = maps == 2 ? launch_sm_mfma_dk<2>(P, dk, dv, grid, stream) : launch_sm_mfma_dk<1>(P, dk, dv, grid, stream);
  if (!ok) abort();   // the caller checks softmax_attention_mfma_supported
}

void launch_headnorm_cache(void* proj, int64_t stride, const int32_t* slots, void* kc, void* vc, int64_t T, int nq,
                           int nk, int dk, int nv, int dv, float eps, const float* qw, const float* kw,
                           const float* bias, const int32_t* pos, float coef, int every, bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    headnorm_cache_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>((float*)proj, stride, slots, (float*)kc,
                                                                       (float*)vc, nq, nk, dk, nv, dv, eps, qw, kw,
                                                                       bias, pos, coef, every);
  else
    headnorm_cache_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)proj, stride, slots,
                                                                          (uint16_t*)kc, (uint16_t*)vc, nq, nk, dk, nv,
                                                                          dv, eps, qw, kw, bias, pos, coef, every);
}

void launch_softmax_attention(void* out, const void* q, int64_t q_stride, const void* gate, int64_t g_stride,
                              const void* kc, const void* vc, const int32_t* block_tables, int max_blocks,
                              const int32_t* tok_seq, const int32_t* pos, int64_t T, int H, int G, int dk, int dv,
                              float scale, int window, int maps, float lam, float unit_eps, float out_scale, bool v_in_k,
                              float softcap, bool f32, hipStream_t stream) {
  if (T == 0) return;
  const int v_row = v_in_k ? dk : dv;
  const dim3 grid((unsigned)T, (unsigned)H);
  const size_t smem = (size_t)(maps * dk + 64) * sizeof(float);
  if (f32)
    softmax_attention_kernel<float><<<grid, 64, smem, stream>>>(
        (float*)out, (const float*)q, q_stride, (const float*)gate, g_stride, (const float*)kc, (const float*)vc,
        block_tables, max_blocks, tok_seq, pos, H, G, dk, dv, scale, window, maps, lam, unit_eps, out_scale, v_row,
        softcap);
  else
    softmax_attention_kernel<uint16_t><<<grid, 64, smem, stream>>>(
        (uint16_t*)out, (const uint16_t*)q, q_stride, (const uint16_t*)gate, g_stride, (const uint16_t*)kc,
        (const uint16_t*)vc, block_tables, max_blocks, tok_seq, pos, H, G, dk, dv, scale, window, maps, lam, unit_eps,
        out_scale, v_row, softcap);
}

}  // namespace nga
