// Gated sigmoid attention over a paged KV cache: un-normalised attention whose weight of a
// visible key is sigmoid(q.k * scale - r1 * ln(1 + r2 * (i - j)) + pb) (r1, r2, pb per query
// head), with a sliding window that also keeps the first tokens of the sequence:
//
//     j visible to i  <=>  j <= i  and  (i - j < window  or  j < keep_first)
//
// and an output gate sigmoid(g) on the concatenated heads. No softmax: no running maximum and
// no normaliser, so key tiles simply accumulate and split sequences need no rescaling.
//
//   qk_norm_cache      per token: RMS-normalise the whole q projection and the whole k
//                      projection (one statistic over all heads, weight per element), write q
//                      back in place and k / v into the token's page slot
//   sigmoid_attention  one wave per (token row, query head), prompt portions and decode rows
//                      alike: keys by lane for q.k, value columns by lane for w.V
//   sigmoid_attention_mfma (bf16)  one workgroup per (64-row block of a sequence, query head):
//                      MFMA q.k and w.V tiles over the pages the block can see
//
// Pages: K [blocks, Hkv, 64, dk], V^T [blocks, Hkv, dv, 64] (T = bf16 or fp32). Scores, the
// distance term, the sigmoid and the accumulation are fp32 in every form.
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

// proj row: [q (Hq*dk) | k (Hkv*dk) | v (Hkv*dv) | ...]; slot < 0: no cache write
template <typename T>
__global__ void __launch_bounds__(256) qk_norm_cache_kernel(T* __restrict__ proj, int64_t stride,
                                                            const float* __restrict__ qw, const float* __restrict__ kw,
                                                            float eps, const int32_t* __restrict__ slots,
                                                            T* __restrict__ kc, T* __restrict__ vc, int Hq, int Hkv,
                                                            int dk, int dv) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  T* pr = proj + row * stride;
  const int nq = Hq * dk, nk = Hkv * dk, nv = Hkv * dv;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq; c += blockDim.x) {
    const float v = ldf(pr + c);
    sq += v * v;
  }
  for (int c = threadIdx.x; c < nk; c += blockDim.x) {
    const float v = ldf(pr + nq + c);
    sk += v * v;
  }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  const float rq = 1.0f / sqrtf(sq / (float)nq + eps);
  const float rk = 1.0f / sqrtf(sk / (float)nk + eps);
  for (int c = threadIdx.x; c < nq; c += blockDim.x) stf(pr + c, ldf(pr + c) * rq * qw[c]);
  const int slot = slots[row];
  if (slot < 0) return;
  const int64_t page = slot / BS;
  const int off = slot % BS;
  for (int c = threadIdx.x; c < nk; c += blockDim.x) {
    const int hh = c / dk, d = c - hh * dk;
    stf(kc + ((page * Hkv + hh) * BS + off) * dk + d, ldf(pr + nq + c) * rk * kw[c]);
  }
  for (int c = threadIdx.x; c < nv; c += blockDim.x) {
    const int hh = c / dv, d = c - hh * dv;
    vc[((page * Hkv + hh) * dv + d) * BS + off] = pr[nq + nk + c];
  }
}

// bf16 rows whose q and k chunks are 16-byte vectors (dk % 8 == 0, nq <= 8192, nk <= 4096): the
// row stays in registers between the two statistics and the write, so it is read once.
__global__ void __launch_bounds__(256) qk_norm_cache_vec_kernel(uint16_t* __restrict__ proj, int64_t stride,
                                                                const float* __restrict__ qw,
                                                                const float* __restrict__ kw, float eps,
                                                                const int32_t* __restrict__ slots,
                                                                uint16_t* __restrict__ kc, uint16_t* __restrict__ vc,
                                                                int Hq, int Hkv, int dk, int dv) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  uint16_t* pr = proj + row * stride;
  const int nq = Hq * dk, nk = Hkv * dk, nv = Hkv * dv;
  const int nq8 = nq / 8, nk8 = nk / 8;
  constexpr int MQ = 4, MK = 2;
  u16x8 qv[MQ], kv[MK];
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int i = 0; i < MQ; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nq8) {
      qv[i] = load8(pr + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) sq += bf2f(qv[i][j]) * bf2f(qv[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < MK; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nk8) {
      kv[i] = load8(pr + nq + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) sk += bf2f(kv[i][j]) * bf2f(kv[i][j]);
    }
  }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  const float rq = 1.0f / sqrtf(sq / (float)nq + eps);
  const float rk = 1.0f / sqrtf(sk / (float)nk + eps);
#pragma unroll
  for (int i = 0; i < MQ; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nq8) {
      u16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = f2bf(bf2f(qv[i][j]) * rq * qw[c * 8 + j]);
      store8(pr + c * 8, o);
    }
  }
  const int slot = slots[row];
  if (slot < 0) return;
  const int64_t page = slot / BS;
  const int off = slot % BS;
#pragma unroll
  for (int i = 0; i < MK; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nk8) {
      const int e = c * 8, hh = e / dk, d = e - hh * dk;
      u16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = f2bf(bf2f(kv[i][j]) * rk * kw[e + j]);
      store8(kc + ((page * Hkv + hh) * BS + off) * dk + d, o);
    }
  }
  for (int c = threadIdx.x; c < nv; c += blockDim.x) {
    const int hh = c / dv, d = c - hh * dv;
    vc[((page * Hkv + hh) * dv + d) * BS + off] = pr[nq + nk + c];
  }
}

// One wave per (token row, head). q: row stride q_stride, head h at h*dk. gate: row stride
// g_stride, head h at h*dv (nullptr: no gate). out [T, Hq*dv].
template <typename T>
__global__ void __launch_bounds__(64) sigmoid_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ gate, int64_t g_stride,
    const T* __restrict__ kc, const T* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int Hq, int Hkv, int dk, int dv,
    float scale, int window, int keep_first, const float* __restrict__ r1, const float* __restrict__ r2,
    const float* __restrict__ pb) {
  extern __shared__ float smem[];
  float* qs = smem;            // [dk]
  float* ws = smem + dk;       // [64]
  const int64_t row = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int i = pos[row];
  T* orow = out + row * (int64_t)Hq * dv + (int64_t)h * dv;
  if (i < 0) {   // padding row
    for (int d = lane; d < dv; d += 64) stf(orow + d, 0.f);
    return;
  }
  const int seq = tok_seq[row];
  const int kvh = h / (Hq / Hkv);
  const int32_t* bt = block_tables + (int64_t)seq * max_blocks;
  for (int d = lane; d < dk; d += 64) qs[d] = ldf(q + row * q_stride + (int64_t)h * dk + d);
  const float a1 = r1[h], a2 = r2[h], b = pb[h];
  constexpr int MAXV = 8;   // dv <= 512
  float acc[MAXV] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int lo = i - window + 1 > 0 ? i - window + 1 : 0;   // first key inside the window
  const int keep = keep_first < lo ? keep_first : lo;        // kept keys [0, keep) below the window
  const int p_keep_end = (keep + BS - 1) / BS;               // pages [0, p_keep_end) hold kept keys
  const int p_lo = lo / BS, p_hi = i / BS;
  __syncthreads();
  for (int p = 0; p <= p_hi; ++p) {
    if (p >= p_keep_end && p < p_lo) {
      p = p_lo - 1;
      continue;
    }
    const int j = p * BS + lane;
    const bool vis = j <= i && (j >= lo || j < keep_first);
    const int64_t page = bt[p];
    float w = 0.f;
    if (vis) {
      const T* kr = kc + ((page * Hkv + kvh) * BS + lane) * dk;
      float s = 0.f;
      for (int d = 0; d < dk; ++d) s += qs[d] * ldf(kr + d);
      s = s * scale - a1 * log1pf(a2 * (float)(i - j));
      w = sigmoidf_(s + b);
    }
    const unsigned long long any = __ballot(vis);
    ws[lane] = w;
    __syncthreads();
    if (any) {
      const int j0 = __builtin_ctzll(any), j1 = 63 - __builtin_clzll(any);
#pragma unroll
      for (int u = 0; u < MAXV; ++u) {
        const int d = lane + u * 64;
        if (d < dv) {
          const T* vr = vc + ((page * Hkv + kvh) * dv + d) * BS;
          float a = acc[u];
          for (int jj = j0; jj <= j1; ++jj) a += ws[jj] * ldf(vr + jj);
          acc[u] = a;
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < MAXV; ++u) {
    const int d = lane + u * 64;
    if (d < dv) {
      float o = acc[u];
      if (gate) o *= sigmoidf_(ldf(gate + row * g_stride + (int64_t)h * dv + d));
      stf(orow + d, o);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// MFMA form for prompt portions (bf16). Workgroup = 4 waves = 64 query rows of one sequence and
// one query head; each wave owns 16 rows, the 16 columns of its mfma_f32_16x16x32_bf16 tiles.
// Per 64-key page the workgroup stages K [64][DK] and V^T [DV][64] in LDS (16-B chunks XOR-
// swizzled by row), then every wave computes S^T = K . Q^T with the key rows permuted so that
// lane (query, h) ends up holding keys 32g + 8h .. + 7 of the page in its accumulators — which is
// exactly the B operand of O^T += V^T . W^T, so the weights never move between lanes. Between
// the two products the weights are formed in fp32 on the VALU (scale, distance term, bias,
// sigmoid, mask). Pages visited: those holding kept first tokens below the block's window, then
// the pages the block's windows cover; everything between is skipped.
__device__ __forceinline__ int sg_row_swz(int row) { return (row & 3) | (((row >> 3) & 3) << 2); }

struct SigMfmaParams {
  uint16_t* out;             // [T, Hq * DV]
  const uint16_t* q;         // row stride q_stride, head h at h * DK
  const uint16_t* gate;      // row stride g_stride, head h at h * DV (nullptr: none)
  const uint16_t* kc;
  const uint16_t* vc;
  const int32_t* block_tables;
  const int32_t* cu_q;       // [B + 1] token rows of each sequence in this launch
  const int32_t* ctx_lens;   // [B] keys of each sequence after this step (its rows are the last ones)
  const float* r1;
  const float* r2;
  const float* pb;
  int64_t q_stride, g_stride;
  int max_blocks, Hq, Hkv, window, keep_first;
  float scale;
};

template <int DK, int DV>
__global__ void __launch_bounds__(256) sigmoid_attention_mfma_kernel(const SigMfmaParams P) {
  constexpr int KT = 64;
  constexpr int NCH_K = DK / 8;
  constexpr int DS = DK / 32;
  constexpr int DT = DV / 16;
  constexpr int PER_K = DK / 32, PER_V = DV / 32;   // 16-B chunks per thread per page
  constexpr int SWS = NCH_K >= 16 ? 0 : NCH_K == 8 ? 1 : 2;
  __shared__ __attribute__((aligned(16))) uint16_t k_s[KT * DK];
  __shared__ __attribute__((aligned(16))) uint16_t v_s[DV * KT];
  // the row block is the slowest grid index and counts down: the blocks that see the most pages
  // are dispatched first for every head and sequence
  const int tile = gridDim.z - 1 - blockIdx.z, hq = blockIdx.x, b = blockIdx.y;
  const int q0 = P.cu_q[b], qlen = P.cu_q[b + 1] - q0;
  if (tile * 64 >= qlen) return;
  const int ctx = P.ctx_lens[b];
  const int kvh = hq / (P.Hq / P.Hkv);
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, h = lane >> 4;
  const int W = P.window, keep = P.keep_first;

  int r = tile * 64 + w * 16 + col;
  const bool row_ok = r < qlen;
  if (!row_ok) r = qlen - 1;
  const int qpos = ctx - qlen + r;
  bf16x8 qf[DS];
  {
    const uint16_t* qp = P.q + (int64_t)(q0 + r) * P.q_stride + (int64_t)hq * DK;
#pragma unroll
    for (int s2 = 0; s2 < DS; ++s2) qf[s2] = as_bf16x8(load8(qp + 32 * s2 + 8 * h));
  }
  // pages of this block: kept ones below its oldest window start, then [t_first, t_last]
  const int qpos_lo = ctx - qlen + tile * 64;
  const int qpos_hi = ctx - qlen + min(qlen - 1, tile * 64 + 63);
  const int lo_min = max(0, qpos_lo - W + 1);
  const int t_first = lo_min / KT, t_last = qpos_hi / KT;
  const int t_keep_end = (min(keep, lo_min) + KT - 1) / KT;
  const float a1 = P.r1[hq], a2 = P.r2[hq];
  constexpr float LOG2E = 1.4426950408889634f;
  const float c0 = -P.scale * LOG2E, c1 = -P.pb[hq] * LOG2E;
  const float fW = (float)W, fkeep = (float)(qpos - keep);   // key < keep  <=>  distance > qpos - keep
  // positions of this wave's first and last valid rows
  const int wq_lo = ctx - qlen + min(qlen - 1, tile * 64 + w * 16);
  const int wq_hi = ctx - qlen + min(qlen - 1, tile * 64 + w * 16 + 15);

  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = (f32x4)(0.f);

  for (int t = 0; t <= t_last; ++t) {
    if (t >= t_keep_end && t < t_first) t = t_first;
    const int64_t blk = P.block_tables[(int64_t)b * P.max_blocks + t];
    const uint16_t* kp = P.kc + (blk * P.Hkv + kvh) * (int64_t)(KT * DK);
    const uint16_t* vp = P.vc + (blk * P.Hkv + kvh) * (int64_t)(DV * KT);
    u16x8 kreg[PER_K], vreg[PER_V];
#pragma unroll
    for (int i = 0; i < PER_K; ++i) kreg[i] = load8(kp + (int64_t)(tid + 256 * i) * 8);
#pragma unroll
    for (int i = 0; i < PER_V; ++i) vreg[i] = load8(vp + (int64_t)(tid + 256 * i) * 8);
    __syncthreads();   // the previous page's reads are done
#pragma unroll
    for (int i = 0; i < PER_K; ++i) {
      const int c = tid + 256 * i;
      const int row = c / NCH_K, ch = c % NCH_K;
      const int sw = sg_row_swz(row) >> SWS;
      *reinterpret_cast<u16x8*>(&k_s[row * DK + ((ch ^ sw) * 8)]) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < PER_V; ++i) {
      const int c = tid + 256 * i;
      const int row = c / 8, ch = c % 8;
      *reinterpret_cast<u16x8*>(&v_s[row * KT + ((ch ^ ((row >> 1) & 7)) * 8)]) = vreg[i];
    }
    __syncthreads();

    f32x4 sacc[4];
#pragma unroll
    for (int tau = 0; tau < 4; ++tau) {
      const int row = 32 * (tau >> 1) + 8 * (col >> 2) + 4 * (tau & 1) + (col & 3);
      const int sw = sg_row_swz(row) >> SWS;
      sacc[tau] = (f32x4)(0.f);
#pragma unroll
      for (int s2 = 0; s2 < DS; ++s2) {
        const int ch = 4 * s2 + h;
        const bf16x8 a = as_bf16x8(*reinterpret_cast<const u16x8*>(&k_s[row * DK + ((ch ^ sw) * 8)]));
        sacc[tau] = mfma16(a, qf[s2], sacc[tau]);
      }
    }
    // weights in the exp2 / log2 domain with the constants folded: sigmoid(z) = 1 / (1 + 2^(-z log2e)),
    // -z log2e = s * c0 + r1 * log2(1 + r2 d) + c1. Distances as floats (exact below 2^24). The
    // mask costs three compares and a select per score and is only applied on pages that cross
    // this wave's diagonal, its window's far edge or the end of the kept prefix (wave-uniform).
    const int kbase = t * KT;
    const float fd = (float)(qpos - kbase - 8 * h);
    const bool need_mask = kbase + KT - 1 > wq_lo || (wq_hi - kbase >= W && kbase + KT > keep);
    bf16x8 pf[2];
#pragma unroll
    for (int tau = 0; tau < 4; ++tau)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const float d = fd - (float)(32 * (tau >> 1) + 4 * (tau & 1) + rr);
        const float lg = __builtin_amdgcn_logf(__builtin_fmaf(a2, d, 1.0f));
        const float zp = __builtin_fmaf(sacc[tau][rr], c0, __builtin_fmaf(a1, lg, c1));
        float wv = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(zp));
        if (need_mask) wv = (d >= 0.f && (d < fW || d > fkeep)) ? wv : 0.f;
        pf[tau >> 1][4 * (tau & 1) + rr] = (__bf16)wv;
      }
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const int ch = 4 * g + h;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const int row = 16 * dt + col;
        const bf16x8 a = as_bf16x8(*reinterpret_cast<const u16x8*>(&v_s[row * KT + ((ch ^ ((row >> 1) & 7)) * 8)]));
        o[dt] = mfma16(a, pf[g], o[dt]);
      }
    }
  }
  if (!row_ok) return;
  uint16_t* op = P.out + (int64_t)(q0 + r) * P.Hq * DV + (int64_t)hq * DV;
  const uint16_t* gp = P.gate ? P.gate + (int64_t)(q0 + r) * P.g_stride + (int64_t)hq * DV : nullptr;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int d = 16 * dt + 4 * h;
    u16x4 ov;
    u16x4 gv;
    if (gp) gv = *reinterpret_cast<const u16x4*>(gp + d);
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      float v = o[dt][rr];
      if (gp) v *= sigmoidf_(bf2f(gv[rr]));
      ov[rr] = f2bf(v);
    }
    *reinterpret_cast<u16x4*>(op + d) = ov;
  }
}

template <int DK>
bool launch_sig_mfma_dv(const SigMfmaParams& P, int dv, dim3 grid, hipStream_t stream) {
  switch (dv) {
    case 32: sigmoid_attention_mfma_kernel<DK, 32><<<grid, 256, 0, stream>>>(P); return true;
    case 64: sigmoid_attention_mfma_kernel<DK, 64><<<grid, 256, 0, stream>>>(P); return true;
    case 128: sigmoid_attention_mfma_kernel<DK, 128><<<grid, 256, 0, stream>>>(P); return true;
    default: return false;
  }
}

// ---------------------------------------------------------------------------------------------
// MFMA form for single-token rows (bf16): the query "columns" of the 16-wide tiles are the query
// heads that share one KV head, so a page is read once for the whole group. Workgroup = 4 waves
// = (token row, KV head, part); every wave walks its own pages of the row's visible list (kept
// pages, then the window's pages), strided over the 4 * parts waves of the row, with the K and
// V^T fragments loaded straight from the page into the MFMA A operands (each byte once, no LDS:
// nothing is shared between waves). Un-normalised weights make partial sums additive: every
// workgroup sums its four waves' fp32 partials [group, DV] through LDS into one workspace slot and
// sigmoid_decode_reduce sums the slots in a fixed order, applies the output gate and writes bf16.
template <int DK, int DV>
__global__ void __launch_bounds__(256) sigmoid_decode_mfma_kernel(
    float* __restrict__ ws, const uint16_t* __restrict__ q, int64_t q_stride, const uint16_t* __restrict__ kc,
    const uint16_t* __restrict__ vc, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ pos, int Hq, int Hkv, float scale, int window,
    int keep_first, const float* __restrict__ r1, const float* __restrict__ r2, const float* __restrict__ pb) {
  constexpr int KT = 64;
  constexpr int DS = DK / 32;
  constexpr int DT = DV / 16;
  const int part = blockIdx.x, parts = gridDim.x, kvh = blockIdx.y;
  const int64_t row = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, h = lane >> 4;
  const int grp = Hq / Hkv;
  const int nslots = parts * 4, slot = part * 4 + w;   // the row's pages are strided over all its waves
  const bool head_ok = col < grp;
  const int hq = kvh * grp + (head_ok ? col : 0);
  const int i = pos[row];

  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = (f32x4)(0.f);
  if (i >= 0) {
    const int32_t* bt = block_tables + (int64_t)tok_seq[row] * max_blocks;
    bf16x8 qf[DS];
    {
      const uint16_t* qp = q + row * q_stride + (int64_t)hq * DK;
#pragma unroll
      for (int s2 = 0; s2 < DS; ++s2) qf[s2] = head_ok ? as_bf16x8(load8(qp + 32 * s2 + 8 * h)) : as_bf16x8((u16x8)(0));
    }
    const float a1 = r1[hq], a2 = r2[hq], bias = pb[hq];
    const int lo = max(0, i - window + 1);
    const int p_lo = lo / KT, p_hi = i / KT;
    const int first_cnt = min((min(keep_first, lo) + KT - 1) / KT, p_lo);   // kept pages below the window's
    const int total = first_cnt + p_hi - p_lo + 1;
    for (int x = slot; x < total; x += nslots) {
      const int t = x < first_cnt ? x : p_lo + (x - first_cnt);
      const int64_t blk = bt[t];
      const uint16_t* kp = kc + (blk * Hkv + kvh) * (int64_t)(KT * DK);
      const uint16_t* vp = vc + (blk * Hkv + kvh) * (int64_t)(DV * KT);
      f32x4 sacc[4];
#pragma unroll
      for (int tau = 0; tau < 4; ++tau) {
        const int krow = 32 * (tau >> 1) + 8 * (col >> 2) + 4 * (tau & 1) + (col & 3);
        sacc[tau] = (f32x4)(0.f);
#pragma unroll
        for (int s2 = 0; s2 < DS; ++s2)
          sacc[tau] = mfma16(as_bf16x8(load8(kp + krow * DK + 32 * s2 + 8 * h)), qf[s2], sacc[tau]);
      }
      const int kbase = t * KT;
      bf16x8 pf[2];
#pragma unroll
      for (int tau = 0; tau < 4; ++tau)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int key = kbase + 32 * (tau >> 1) + 8 * h + 4 * (tau & 1) + rr;
          const int dist = i - key;
          const bool ok = dist >= 0 && (dist < window || key < keep_first);
          const float z = sacc[tau][rr] * scale - a1 * __logf(1.0f + a2 * (float)dist) + bias;
          const float wv = ok ? __builtin_amdgcn_rcpf(1.0f + __expf(-z)) : 0.f;
          pf[tau >> 1][4 * (tau & 1) + rr] = (__bf16)wv;
        }
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          o[dt] = mfma16(as_bf16x8(load8(vp + (16 * dt + col) * KT + 32 * g + 8 * h)), pf[g], o[dt]);
    }
  }
  // the workgroup's four partials -> one slot: through LDS, summed in wave order
  __shared__ float red_s[4][DV][17];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) red_s[w][16 * dt + 4 * h + rr][col] = o[dt][rr];
  __syncthreads();
  for (int e = tid; e < grp * DV; e += 256) {
    const int c = e / DV, d = e - c * DV;
    const float sum = ((red_s[0][d][c] + red_s[1][d][c]) + red_s[2][d][c]) + red_s[3][d][c];
    ws[((row * Hq + kvh * grp + c) * parts + part) * (int64_t)DV + d] = sum;
  }
}

// out[row, hq*dv + d] = (sum over slots of ws[row, hq, slot, d]) * sigmoid(gate)
__global__ void __launch_bounds__(256) sigmoid_decode_reduce_kernel(uint16_t* __restrict__ out,
                                                                    const float* __restrict__ ws,
                                                                    const uint16_t* __restrict__ gate,
                                                                    int64_t g_stride, int64_t total, int HD, int dv,
                                                                    int nslots) {
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = e / HD;
    const int c = (int)(e - row * HD);
    const int hq = c / dv, d = c - hq * dv;
    const float* wp = ws + ((row * (HD / dv) + hq) * nslots) * (int64_t)dv + d;
    float acc = 0.f;
    for (int sl = 0; sl < nslots; ++sl) acc += wp[(int64_t)sl * dv];
    if (gate) acc *= sigmoidf_(bf2f(gate[row * g_stride + c]));
    out[e] = f2bf(acc);
  }
}

template <int DK>
bool launch_sig_decode_dv(int dv, dim3 grid, hipStream_t stream, float* ws, const uint16_t* q, int64_t q_stride,
                          const uint16_t* kc, const uint16_t* vc, const int32_t* bt, int max_blocks,
                          const int32_t* tok_seq, const int32_t* pos, int Hq, int Hkv, float scale, int window,
                          int keep_first, const float* r1, const float* r2, const float* pb) {
#define NGA_SIG_DEC(DV_)                                                                                             \
  sigmoid_decode_mfma_kernel<DK, DV_><<<grid, 256, 0, stream>>>(ws, q, q_stride, kc, vc, bt, max_blocks, tok_seq, pos, \
                                                                Hq, Hkv, scale, window, keep_first, r1, r2, pb)
  switch (dv) {
    case 32: NGA_SIG_DEC(32); return true;
    case 64: NGA_SIG_DEC(64); return true;
    case 128: NGA_SIG_DEC(128); return true;
    default: return false;
  }
#undef NGA_SIG_DEC
}

}  // namespace

void launch_qk_norm_cache(void* proj, int64_t stride, const float* qw, const float* kw, float eps,
                          const int32_t* slots, void* kc, void* vc, int64_t T, int Hq, int Hkv, int dk, int dv,
                          bool f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    qk_norm_cache_kernel<float><<<dim3((unsigned)T), 256, 0, stream>>>((float*)proj, stride, qw, kw, eps, slots,
                                                                      (float*)kc, (float*)vc, Hq, Hkv, dk, dv);
  else if (dk % 8 == 0 && stride % 8 == 0 && Hq * dk <= 8192 && Hkv * dk <= 4096 &&
           ((uintptr_t)proj | (uintptr_t)kc) % 16 == 0)
    qk_norm_cache_vec_kernel<<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)proj, stride, qw, kw, eps, slots,
                                                                   (uint16_t*)kc, (uint16_t*)vc, Hq, Hkv, dk, dv);
  else
    qk_norm_cache_kernel<uint16_t><<<dim3((unsigned)T), 256, 0, stream>>>((uint16_t*)proj, stride, qw, kw, eps, slots,
                                                                         (uint16_t*)kc, (uint16_t*)vc, Hq, Hkv, dk,
                                                                         dv);
}

void launch_sigmoid_attention(void* out, const void* q, int64_t q_stride, const void* gate, int64_t g_stride,
                              const void* kc, const void* vc, const int32_t* block_tables, int max_blocks,
                              const int32_t* tok_seq, const int32_t* pos, int64_t T, int Hq, int Hkv, int dk, int dv,
                              float scale, int window, int keep_first, const float* r1, const float* r2,
                              const float* pb, bool f32, hipStream_t stream) {
  if (T == 0) return;
  const dim3 grid((unsigned)T, (unsigned)Hq);
  const size_t lds = (size_t)(dk + 64) * sizeof(float);
  if (f32)
    sigmoid_attention_kernel<float><<<grid, 64, lds, stream>>>(
        (float*)out, (const float*)q, q_stride, (const float*)gate, g_stride, (const float*)kc, (const float*)vc,
        block_tables, max_blocks, tok_seq, pos, Hq, Hkv, dk, dv, scale, window, keep_first, r1, r2, pb);
  else
    sigmoid_attention_kernel<uint16_t><<<grid, 64, lds, stream>>>(
        (uint16_t*)out, (const uint16_t*)q, q_stride, (const uint16_t*)gate, g_stride, (const uint16_t*)kc,
        (const uint16_t*)vc, block_tables, max_blocks, tok_seq, pos, Hq, Hkv, dk, dv, scale, window, keep_first, r1,
        r2, pb);
}

bool sigmoid_attention_mfma_supported(int dk, int dv) {
  return (dk == 32 || dk == 64 || dk == 128) && (dv == 32 || dv == 64 || dv == 128);
}

// Prompt portions on the MFMA kernel: sequence b owns token rows [cu_q[b], cu_q[b + 1]), the last
// ones of its ctx_lens[b] keys. Row strides and the gate pointer must be 8-byte aligned (checked
// by the caller together with sigmoid_attention_mfma_supported).
void launch_sigmoid_attention_mfma(uint16_t* out, const uint16_t* q, int64_t q_stride, const uint16_t* gate,
                                   int64_t g_stride, const uint16_t* kc, const uint16_t* vc,
                                   const int32_t* block_tables, int max_blocks, const int32_t* cu_q,
                                   const int32_t* ctx_lens, int B, int max_q_len, int Hq, int Hkv, int dk, int dv,
                                   float scale, int window, int keep_first, const float* r1, const float* r2,
                                   const float* pb, hipStream_t stream) {
  if (B == 0 || max_q_len == 0) return;
  SigMfmaParams P{out, q, gate, kc, vc, block_tables, cu_q, ctx_lens, r1, r2, pb, q_stride, g_stride,
                  max_blocks, Hq, Hkv, window, keep_first, scale};
  const dim3 grid((unsigned)Hq, (unsigned)B, (unsigned)((max_q_len + 63) / 64));   // (head, sequence, row block)
  bool ok = false;
  if (dk == 32) ok = launch_sig_mfma_dv<32>(P, dv, grid, stream);
  else if (dk == 64) ok = launch_sig_mfma_dv<64>(P, dv, grid, stream);
  else if (dk == 128) ok = launch_sig_mfma_dv<128>(P, dv, grid, stream);
  if (!ok) abort();   // the caller checks sigmoid_attention_mfma_supported
}

// Parts (workgroups per row and KV head) of the single-token MFMA kernel: enough waves to fill
// the chip, never more than the pages a row can see. Fixed by sizes the host knows, so a
// captured step keeps its launch shape.
int sigmoid_decode_parts(int rows, int Hkv, int max_ctx, int window, int keep_first) {
  const int64_t span = (int64_t)window + keep_first;
  const int pages = (int)((span < max_ctx ? span : max_ctx) / 64) + 2;
  int by_pages = (pages + 3) / 4;
  int target = kernel_form(KF_SIG_DECODE_WAVES);   // waves to launch: 8192 = 8 per SIMD on 256 CUs
  if (target < 1) target = 1;
  int by_fill = (target + rows * Hkv * 4 - 1) / (rows * Hkv * 4);
  int p = by_pages < by_fill ? by_pages : by_fill;
  return p < 1 ? 1 : (p > 64 ? 64 : p);
}

// ws: fp32 [T, Hq, parts, dv]
void launch_sigmoid_decode_mfma(uint16_t* out, float* ws, int parts, const uint16_t* q, int64_t q_stride,
                                const uint16_t* gate, int64_t g_stride, const uint16_t* kc, const uint16_t* vc,
                                const int32_t* block_tables, int max_blocks, const int32_t* tok_seq,
                                const int32_t* pos, int64_t T, int Hq, int Hkv, int dk, int dv, float scale,
                                int window, int keep_first, const float* r1, const float* r2, const float* pb,
                                hipStream_t stream) {
  if (T == 0) return;
  const dim3 grid((unsigned)parts, (unsigned)Hkv, (unsigned)T);
  bool ok = false;
#define NGA_SIG_ARGS dv, grid, stream, ws, q, q_stride, kc, vc, block_tables, max_blocks, tok_seq, pos, Hq, Hkv, scale, \
                     window, keep_first, r1, r2, pb
  if (dk == 32) ok = launch_sig_decode_dv<32>(NGA_SIG_ARGS);
  else if (dk == 64) ok = launch_sig_decode_dv<64>(NGA_SIG_ARGS);
  else if (dk == 128) ok = launch_sig_decode_dv<128>(NGA_SIG_ARGS);
#undef NGA_SIG_ARGS
  if (!ok) abort();   // the caller checks sigmoid_attention_mfma_supported
  const int64_t total = T * Hq * dv;
  int64_t g = (total + 255) / 256;
  if (g > 4096) g = 4096;
  sigmoid_decode_reduce_kernel<<<dim3((unsigned)g), 256, 0, stream>>>(out, ws, gate, g_stride, total, Hq * dv, dv,
                                                                     parts);
}

}  // namespace nga
