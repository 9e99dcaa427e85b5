// Many small matrix products in one launch, C_g = A_g . W_g^T, and what a routed feed-forward needs around them.
//
// Two ways of naming the groups:
//   heads    group z is a head: A_z, W_z and C_z are column blocks / slabs at fixed strides (a_zs, w_zs, c_zs) and all
//            groups have the same M rows. With `gate`, row m of C_z is multiplied by sigmoid(gate[m, z]).
//   experts  group g is an expert: its rows are the entries offsets[g] .. offsets[g+1] of a list sorted by expert
//            (`perm`: sorted place -> entry = token * top + choice). A row is read either from the entry's token
//            (a_div = top: the gate and up projections read the step's rows) or from the sorted place itself
//            (a_div = 0: the down projection reads what the first product left), and written to the sorted place
//            or, with c_to_perm, to the entry. The work list `tiles` names (expert, first sorted place) of every
//            row tile; entries beyond the step's tiles hold -1 and their workgroups leave at once.
// GATED: W_g = [gate rows; up rows] stacked, gate_n rows each, and C = silu(A Wgate^T) * (A Wup^T).
//
// Float operands run on the vector ALUs, every output element summed over k in ascending order by one thread (the
// true 32-bit path; a row's result does not depend on which tile or group size it met). bf16 operands run on the
// matrix cores, operands read straight from memory in the MFMA's own order (8 consecutive k a lane), in two forms:
// tiles of 128 rows (a wave 64 x 64 outputs) and tiles of 16 rows whose waves split k (see the kernels).
//
//   moe_route    two kernels: router logits in float (a wave an expert, a router row read once per 8 tokens), then per
//                token the `top` largest (lowest index first among equals), the softmax over the chosen and the shared
//                expert's sigmoid gate
//   moe_scatter  counts, offsets, the sorted list and the work list, one workgroup (LDS counters)
//   moe_combine  out[t] = sum_c share[t, c] * y[t * top + c] + shared_gate[t] * shared[t]   (no gate: + shared[t])
#include "common.cuh"

using namespace dinfer;

namespace {

struct Groups {
  const void* A; int64_t lda, a_zs;
  const void* W; int64_t ldw, w_zs;
  void* C; int64_t ldc, c_zs;
  int M, N, K;
  const int32_t* tiles;     // experts: [max_tiles][2]
  const int32_t* offsets;   // experts: [G + 1]
  const int32_t* perm;      // experts: sorted place -> entry
  int a_div;                // experts: > 0: A row = perm[i] / a_div; 0: A row = i
  int c_to_perm;            // experts: C row = perm[i] instead of i
  const void* gate; int64_t ld_gate;   // heads: optional
  int gate_n;               // GATED: rows of each half of W_g
  int tm;                   // rows of a tile: 64 on the vector ALUs, 16 or 128 on the matrix cores
  int act;                  // not GATED: 0 nothing, 1 silu, 2 gelu (error function) on every result
};

__device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float plain_act(float x, int act) {
  if (act == 1) return silu(x);
  if (act == 2) return 0.5f * x * (1.f + erff(x * 0.7071067811865476f));
  return x;
}

constexpr int BM = 64, BN = 64, BK = 16;

// Which rows this workgroup's tile holds: group z, local rows [m0, m0 + rows), and for local row r the rows of A and C.
struct Tile {
  int z, m0, rows;
  const int32_t* perm; int a_div, c_to_perm, base;
  __device__ __forceinline__ bool init(const Groups& p) {
    const int tm = p.tm;   // rows a tile
    if (p.tiles) {
      z = p.tiles[2 * blockIdx.y];
      if (z < 0) return false;
      base = p.tiles[2 * blockIdx.y + 1];
      m0 = 0;
      const int end = p.offsets[z + 1];
      rows = end - base < tm ? end - base : tm;
      perm = p.perm; a_div = p.a_div; c_to_perm = p.c_to_perm;
    } else {
      z = blockIdx.z;
      m0 = blockIdx.y * tm;
      rows = p.M - m0 < tm ? p.M - m0 : tm;
      perm = nullptr; a_div = 0; c_to_perm = 0; base = m0;
    }
    return rows > 0;
  }
  __device__ __forceinline__ int64_t a_row(int r) const { return perm && a_div > 0 ? perm[base + r] / a_div : base + r; }
  __device__ __forceinline__ int64_t c_row(int r) const { return perm && c_to_perm ? perm[base + r] : base + r; }
};

template <class S, class O, bool GATED>
__global__ void __launch_bounds__(256) grouped_valu_kernel(Groups p) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  __shared__ float Us[GATED ? BK : 1][BN + 4];
  __shared__ int64_t arow[BM];
  Tile tl;
  if (!tl.init(p)) return;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int n0 = blockIdx.x * BN;
  const bool experts = p.tiles != nullptr;
  const S* A = (const S*)p.A + (experts ? 0 : (int64_t)tl.z * p.a_zs);
  const S* W = (const S*)p.W + (int64_t)tl.z * p.w_zs;
  if (threadIdx.x < BM) arow[threadIdx.x] = threadIdx.x < tl.rows ? tl.a_row(threadIdx.x) : -1;
  __syncthreads();
  float acc[4][4], acu[GATED ? 4 : 1][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = 0.f;
      if (GATED) acu[i][j] = 0.f;
    }
  for (int k0 = 0; k0 < p.K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = e * 256 + threadIdx.x;
      const int r = idx >> 4, kk = idx & 15;
      const int gk = k0 + kk, gn = n0 + r;
      const int64_t ar = arow[r];
      As[kk][r] = (ar >= 0 && gk < p.K) ? to_f32(A[ar * p.lda + gk]) : 0.f;
      Ws[kk][r] = (gn < p.N && gk < p.K) ? to_f32(W[(int64_t)gn * p.ldw + gk]) : 0.f;
      if (GATED) Us[kk][r] = (gn < p.N && gk < p.K) ? to_f32(W[(int64_t)(gn + p.gate_n) * p.ldw + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], w[4], u[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        w[j] = Ws[kk][tx * 4 + j];
        if (GATED) u[j] = Us[kk][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
          if (GATED) acu[i][j] = fmaf(a[i], u[j], acu[i][j]);
        }
    }
    __syncthreads();
  }
  O* C = (O*)p.C + (experts ? 0 : (int64_t)tl.z * p.c_zs);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= tl.rows) continue;
    const int64_t cr = tl.c_row(r);
    float g = 1.f;
    if (p.gate) g = sigmoid(to_f32(((const S*)p.gate)[cr * p.ld_gate + tl.z]));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < p.N) {
        float v = GATED ? silu(acc[i][j]) * acu[i][j] : plain_act(acc[i][j], p.act);
        C[cr * p.ldc + gn] = from_f32<O>(v * g);
      }
    }
  }
}

// bf16 on the matrix cores. v_mfma_f32_16x16x32_bf16: lane l holds row (or column) l % 16 and the 8 consecutive k
// starting at 8 (l / 16); of the result it holds column l % 16, rows 4 (l / 16) .. + 3. Operands are read straight from
// memory in that order (16 bytes a lane).
//
// Many rows (tiles of 128): a workgroup takes 128 rows x 128 columns (gated: 64 columns of each half), its waves
// 2 x 2, a wave 64 x 64. Both operands are staged through LDS 64 k at a time (16-byte pieces, read from memory by
// the whole workgroup once, rows gathered through the tile's row list on the way), the next step's pieces are loaded
// into registers while this step is multiplied; four row fragments and four column fragments feed sixteen MFMAs per
// 32 k. Every output element is still summed over ascending k by one lane.
constexpr int TM_BIG = 128, TM_SMALL = 16;

constexpr int BIG_K = 64;            // k a step
constexpr int BIG_LD = BIG_K + 8;    // row of a staged tile in LDS, padded: rows 16 bytes apart in the banks

template <class O, bool GATED>
__global__ void __launch_bounds__(256) grouped_mfma_big_kernel(Groups p) {
  __shared__ int64_t arow[TM_BIG];
  __shared__ __attribute__((aligned(16))) bf16 As[TM_BIG * BIG_LD];
  __shared__ __attribute__((aligned(16))) bf16 Ws[128 * BIG_LD];
  Tile tl;
  if (!tl.init(p)) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int n0 = blockIdx.x * (GATED ? 64 : 128);
  const bool experts = p.tiles != nullptr;
  const bf16* A = (const bf16*)p.A + (experts ? 0 : (int64_t)tl.z * p.a_zs);
  const bf16* W = (const bf16*)p.W + (int64_t)tl.z * p.w_zs;
  if (threadIdx.x < TM_BIG) arow[threadIdx.x] = threadIdx.x < tl.rows ? tl.a_row(threadIdx.x) : -1;
  __syncthreads();
  // staging: a tile is 128 rows x 64 k = 1,024 pieces of 16 bytes, four a thread for each operand; piece q of a thread
  // is row (q * 256 + thread) / 8, k piece (thread % 8)
  const int sp = threadIdx.x & 7;
  const bf16* ag[4];
  const bf16* wg[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int row = (q * 256 + threadIdx.x) >> 3;
    const int64_t ar = arow[row];
    ag[q] = ar >= 0 ? A + ar * p.lda + sp * 8 : nullptr;
    // row of the weight behind row `row` of the staged tile; gated: 64 gate rows, then the 64 up rows of the same numbers
    const int gn = GATED ? n0 + (row & 63) : n0 + row;
    const int64_t wrow = GATED && row >= 64 ? gn + p.gate_n : gn;
    wg[q] = gn < p.N ? W + wrow * p.ldw + sp * 8 : nullptr;
  }
  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
  const int K = p.K;   // a multiple of 8 (checked on the host)
  bf16x8 an[4], wn_[4];
  auto fetch = [&](int k0) {
    const bool in = k0 + sp * 8 < K;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      an[q] = (ag[q] && in) ? *(const bf16x8*)(ag[q] + k0) : zero;
      wn_[q] = (wg[q] && in) ? *(const bf16x8*)(wg[q] + k0) : zero;
    }
  };
  const int lr = lane & 15, kq = lane >> 4;
  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BIG_K) {
    __syncthreads();      // the step before has read the tiles
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row = (q * 256 + threadIdx.x) >> 3;
      *(bf16x8*)(As + row * BIG_LD + sp * 8) = an[q];
      *(bf16x8*)(Ws + row * BIG_LD + sp * 8) = wn_[q];
    }
    __syncthreads();
    if (k0 + BIG_K < K) fetch(k0 + BIG_K);    // the next step's pieces travel while this one is multiplied
#pragma unroll
    for (int kk = 0; kk < BIG_K; kk += 32) {
      bf16x8 a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = *(const bf16x8*)(As + (wm * 64 + i * 16 + lr) * BIG_LD + kk + kq * 8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // gated: fragments 0, 1 are gate columns, 2, 3 the up columns of the same numbers
        const int row = GATED ? (j >> 1) * 64 + wn * 32 + (j & 1) * 16 + lr : wn * 64 + j * 16 + lr;
        w[j] = *(const bf16x8*)(Ws + row * BIG_LD + kk + kq * 8);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], w[j], acc[i][j], 0, 0, 0);
    }
  }
  O* C = (O*)p.C + (experts ? 0 : (int64_t)tl.z * p.c_zs);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = wm * 64 + i * 16 + kq * 4 + r;
      if (row >= tl.rows) continue;
      const int64_t cr = tl.c_row(row);
      float g = 1.f;
      if (p.gate) g = sigmoid((float)((const bf16*)p.gate)[cr * p.ld_gate + tl.z]);
#pragma unroll
      for (int j = 0; j < (GATED ? 2 : 4); ++j) {
        const int gn = GATED ? n0 + wn * 32 + j * 16 + lr : n0 + wn * 64 + j * 16 + lr;
        if (gn < p.N) {
          const float v = GATED ? silu(acc[i][j][r]) * acc[i][j + 2][r] : plain_act(acc[i][j][r], p.act);
          C[cr * p.ldc + gn] = from_f32<O>(v * g);
        }
      }
    }
}

// Few rows (tiles of 16: steps of single tokens): time is the time to stream the weights, so a workgroup takes only 16
// columns (gated: of each half) and its four waves take a quarter of k each; their partial sums meet in LDS and are
// added in wave order.
template <class O, bool GATED>
__global__ void __launch_bounds__(256) grouped_mfma_small_kernel(Groups p) {
  __shared__ int64_t arow[TM_SMALL];
  __shared__ float part[4][GATED ? 2 : 1][16][17];
  Tile tl;
  if (!tl.init(p)) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n0 = blockIdx.x * 16;
  const bool experts = p.tiles != nullptr;
  const bf16* A = (const bf16*)p.A + (experts ? 0 : (int64_t)tl.z * p.a_zs);
  const bf16* W = (const bf16*)p.W + (int64_t)tl.z * p.w_zs;
  if (threadIdx.x < TM_SMALL) arow[threadIdx.x] = threadIdx.x < tl.rows ? tl.a_row(threadIdx.x) : -1;
  __syncthreads();
  const int lr = lane & 15, kq = lane >> 4;
  const int64_t ar = arow[lr];
  const int gn = n0 + lr;
  const bf16* ap = ar >= 0 ? A + ar * p.lda + kq * 8 : nullptr;
  const bf16* wp = gn < p.N ? W + (int64_t)gn * p.ldw + kq * 8 : nullptr;
  const bf16* up = (GATED && gn < p.N) ? W + (int64_t)(gn + p.gate_n) * p.ldw + kq * 8 : nullptr;
  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
  const int K = p.K;
  const int steps = (K + 31) / 32, per = (steps + 3) / 4;
  const int k_lo = wave * per * 32, k_hi = (wave + 1) * per * 32 < K ? (wave + 1) * per * 32 : K;
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f}, acu = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k0 = k_lo; k0 < k_hi; k0 += 32) {
    const bool in = k0 + kq * 8 < K;
    const bf16x8 a = (ap && in) ? *(const bf16x8*)(ap + k0) : zero;
    const bf16x8 w = (wp && in) ? __builtin_nontemporal_load((const bf16x8*)(wp + k0)) : zero;
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, w, acc, 0, 0, 0);
    if (GATED) {
      const bf16x8 u = (up && in) ? __builtin_nontemporal_load((const bf16x8*)(up + k0)) : zero;
      acu = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, u, acu, 0, 0, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    part[wave][0][kq * 4 + r][lr] = acc[r];
    if (GATED) part[wave][GATED ? 1 : 0][kq * 4 + r][lr] = acu[r];
  }
  __syncthreads();
  const int row = threadIdx.x >> 4, col = threadIdx.x & 15;
  if (row >= tl.rows || n0 + col >= p.N) return;
  float v = 0.f, u = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    v += part[w][0][row][col];
    if (GATED) u += part[w][GATED ? 1 : 0][row][col];
  }
  const int64_t cr = tl.c_row(row);
  float g = 1.f;
  if (p.gate) g = sigmoid((float)((const bf16*)p.gate)[cr * p.ld_gate + tl.z]);
  O* C = (O*)p.C + (experts ? 0 : (int64_t)tl.z * p.c_zs);
  C[cr * p.ldc + n0 + col] = from_f32<O>((GATED ? silu(v) * u : plain_act(v, p.act)) * g);
}

// ---- routing ---------------------------------------------------------------------------------------------------
constexpr int MAX_EXPERTS = 1024;

// Router logits: a wave takes one expert (the row after the last expert is the shared expert's gate vector) and up to
// RT tokens (8 in steps of many tokens, so that a router row is read once per 8; 1 in steps of few, where more
// workgroups matter more); a lane sums every 64th entry, then the lanes meet. z [T, ldz].
template <class S, int RT>
__global__ void __launch_bounds__(256) moe_logits_kernel(const S* __restrict__ x, int64_t ld_x, int tokens,
                                                         const float* __restrict__ wr, const float* __restrict__ wsg,
                                                         int E, int width, float* __restrict__ z, int ldz) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e = blockIdx.y * 4 + wave;
  if (e >= E + (wsg ? 1 : 0)) return;
  const float* w = e < E ? wr + (int64_t)e * width : wsg;
  const int t0 = blockIdx.x * RT;
  const int nt = tokens - t0 < RT ? tokens - t0 : RT;
  float acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = 0.f;
#pragma unroll 4
  for (int i = lane; i < width; i += 64) {
    const float wv = w[i];
#pragma unroll
    for (int r = 0; r < RT; ++r)
      if (r < nt) acc[r] = fmaf(to_f32(x[(int64_t)(t0 + r) * ld_x + i]), wv, acc[r]);
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const float v = wave_sum(acc[r]);
    if (lane == 0 && r < nt) z[(int64_t)(t0 + r) * ldz + e] = v;
  }
}

// The same for bfloat16 rows of a width that is a multiple of 8: a lane takes 8 consecutive entries at a time (16-byte
// loads of x, two of the router's row), so a token costs an eighth of the load instructions.
template <int RT>
__global__ void __launch_bounds__(256) moe_logits_bf16x8_kernel(const bf16* __restrict__ x, int64_t ld_x, int tokens,
                                                                const float* __restrict__ wr, const float* __restrict__ wsg,
                                                                int E, int width, float* __restrict__ z, int ldz) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int e = blockIdx.y * 4 + wave;
  if (e >= E + (wsg ? 1 : 0)) return;
  const float* w = e < E ? wr + (int64_t)e * width : wsg;
  const int t0 = blockIdx.x * RT;
  const int nt = tokens - t0 < RT ? tokens - t0 : RT;
  float acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = 0.f;
  for (int i = lane * 8; i < width; i += 512) {
    const f32x4 w0 = *(const f32x4*)(w + i), w1 = *(const f32x4*)(w + i + 4);
#pragma unroll
    for (int r = 0; r < RT; ++r)
      if (r < nt) {
        const bf16x8 v = *(const bf16x8*)(x + (int64_t)(t0 + r) * ld_x + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[r] = fmaf((float)v[j], w0[j], acc[r]);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[r] = fmaf((float)v[4 + j], w1[j], acc[r]);
      }
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const float v = wave_sum(acc[r]);
    if (lane == 0 && r < nt) z[(int64_t)(t0 + r) * ldz + e] = v;
  }
}

// A wave per token: the `top` largest of its logits, one after the other (among equals the lowest index), the softmax
// over the chosen, and the sigmoid of the shared expert's gate logit (z[t, E]) where there is one.
// all_scores: the scores are the softmax over all E logits; the choice goes by score + correction[e] (correction may
// be null) and a chosen expert's weight is its score as it is (the weights of a token need not sum to one).
__global__ void __launch_bounds__(256) moe_topk_kernel(const float* __restrict__ z, int ldz, int tokens, int E, int top,
                                                       int has_shared, int32_t* __restrict__ idx,
                                                       float* __restrict__ share, float* __restrict__ shared_gate,
                                                       int all_scores, const float* __restrict__ correction) {
  __shared__ float zs[4][MAX_EXPERTS];
  __shared__ float sc[4][MAX_EXPERTS];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + wave;
  if (t >= tokens) return;   // (no workgroup barrier below)
  float* zw = zs[wave];
  for (int e = lane; e < E; e += 64) zw[e] = z[t * ldz + e];
  if (has_shared && lane == 0) shared_gate[t] = sigmoid(z[t * ldz + E]);
  if (all_scores) {
    float* sw = sc[wave];
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, zw[e]);   // (a lane reads back what it wrote itself)
    mx = wave_max(mx);
    float den = 0.f;
    for (int e = lane; e < E; e += 64) { const float p = expf(zw[e] - mx); sw[e] = p; den += p; }
    den = wave_sum(den);
    for (int e = lane; e < E; e += 64) {
      const float p = sw[e] / den;
      sw[e] = p;
      zw[e] = p + (correction ? correction[e] : 0.f);
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    int chosen_e = 0;
    for (int c = 0; c < top; ++c) {
      float best = -INFINITY;
      int be = 0x7fffffff;
      for (int e = lane; e < E; e += 64) {
        const float v = zw[e];
        if (v > best || (v == best && e < be)) { best = v; be = e; }
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oe = __shfl_xor(be, o, 64);
        if (ov > best || (ov == best && oe < be)) { best = ov; be = oe; }
      }
      if (lane == c) chosen_e = be;
      if (lane == 0 && be < E) zw[be] = -INFINITY;
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    if (lane < top) {
      idx[t * top + lane] = chosen_e;
      share[t * top + lane] = chosen_e < E ? sw[chosen_e] : 0.f;
    }
    return;
  }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
  float chosen = 0.f, zmax = 0.f, sum = 0.f;   // lane c keeps the c-th choice
  int chosen_e = 0;
  for (int c = 0; c < top; ++c) {
    float best = -INFINITY;
    int be = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = zw[e];
      if (v > best || (v == best && e < be)) { best = v; be = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      if (ov > best || (ov == best && oe < be)) { best = ov; be = oe; }
    }
    if (c == 0) zmax = best;
    if (lane == c) { chosen = best; chosen_e = be; }
    if (lane == 0 && be < E) zw[be] = -INFINITY;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    sum += expf(best - zmax);   // every lane holds the same sum, added in the order of the choices
  }
  if (lane < top) {
    idx[t * top + lane] = chosen_e;
    share[t * top + lane] = expf(chosen - zmax) / sum;
  }
}

// One workgroup. entries = tokens * top.
// Experts from `real` on have no weights (their output is their input): their entries are sorted like the others', but
// no tile is made for them.
__global__ void __launch_bounds__(1024) moe_scatter_kernel(const int32_t* __restrict__ idx, int entries, int E, int tile_rows,
                                                           int32_t* __restrict__ offsets, int32_t* __restrict__ perm,
                                                           int32_t* __restrict__ tiles, int max_tiles, int real) {
  __shared__ int cnt[MAX_EXPERTS], off[MAX_EXPERTS + 1], tbase[MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < entries; i += blockDim.x) atomicAdd(&cnt[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int o = 0, tb = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = o; tbase[e] = tb;
      o += cnt[e];
      if (e < real) tb += (cnt[e] + tile_rows - 1) / tile_rows;
    }
    off[E] = o; tbase[E] = tb;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = off[e];
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    const int n = tbase[e + 1] - tbase[e];
    for (int k = 0; k < n; ++k) {
      const int at = tbase[e] + k;
      if (at < max_tiles) { tiles[2 * at] = e; tiles[2 * at + 1] = off[e] + k * tile_rows; }
    }
    cnt[e] = 0;   // now the cursor
  }
  for (int at = tbase[E] + threadIdx.x; at < max_tiles; at += blockDim.x) { tiles[2 * at] = -1; tiles[2 * at + 1] = 0; }
  __syncthreads();
  for (int i = threadIdx.x; i < entries; i += blockDim.x) {
    const int e = idx[i];
    perm[off[e] + atomicAdd(&cnt[e], 1)] = i;
  }
}

template <class S>
__global__ void __launch_bounds__(256) moe_combine_kernel(const S* __restrict__ y, int64_t ld_y, const float* __restrict__ share,
                                                          int top, const S* __restrict__ shared, int64_t ld_s,
                                                          const float* __restrict__ shared_gate, S* __restrict__ out,
                                                          int64_t ld_o, int width, const int32_t* __restrict__ idx,
                                                          int real, const S* __restrict__ x, int64_t ld_x) {
  const int64_t t = blockIdx.x;
  const float sg = shared ? (shared_gate ? shared_gate[t] : 1.f) : 0.f;   // no gate: the shared output as it is
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float acc = 0.f;
    for (int c = 0; c < top; ++c) {
      // an expert without weights hands the token's input on
      const bool same = idx && idx[t * top + c] >= real;
      acc = fmaf(share[t * top + c], to_f32(same ? x[t * ld_x + i] : y[(t * top + c) * ld_y + i]), acc);
    }
    if (shared) acc = fmaf(sg, to_f32(shared[t * ld_s + i]), acc);
    out[t * ld_o + i] = from_f32<S>(acc);
  }
}

inline bool mfma_fits(int dtype, const Groups& p) {
  return dtype == DT_BF16 && p.K % 8 == 0 && p.lda % 8 == 0 && p.ldw % 8 == 0 && p.a_zs % 8 == 0 && p.w_zs % 8 == 0 &&
         ((uintptr_t)p.A % 16) == 0 && ((uintptr_t)p.W % 16) == 0;
}

// grid.x is set here from the kernel's columns a workgroup; grid.y / z arrive from the caller (tiles, groups).
// bf16 rows whose width is a multiple of 8: a thread takes 8 consecutive entries of every chosen expert's row.
__global__ void __launch_bounds__(256) moe_combine_bf16x8_kernel(const bf16* __restrict__ y, int64_t ld_y,
                                                                 const float* __restrict__ share, int top,
                                                                 const bf16* __restrict__ shared, int64_t ld_s,
                                                                 const float* __restrict__ shared_gate,
                                                                 bf16* __restrict__ out, int64_t ld_o, int width,
                                                                 const int32_t* __restrict__ idx, int real,
                                                                 const bf16* __restrict__ x, int64_t ld_x) {
  const int64_t t = blockIdx.x;
  const float sg = shared ? (shared_gate ? shared_gate[t] : 1.f) : 0.f;   // no gate: the shared output as it is
  for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    for (int c = 0; c < top; ++c) {
      const bool same = idx && idx[t * top + c] >= real;   // an expert without weights hands the token's input on
      const bf16x8 v = *(const bf16x8*)(same ? x + t * ld_x + i : y + (t * top + c) * ld_y + i);
      const float w = share[t * top + c];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = fmaf(w, (float)v[j], acc[j]);
    }
    if (shared) {
      const bf16x8 v = *(const bf16x8*)(shared + t * ld_s + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = fmaf(sg, (float)v[j], acc[j]);
    }
    bf16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (bf16)acc[j];
    *(bf16x8*)(out + t * ld_o + i) = r;
  }
}

template <bool GATED>
int launch_groups(int dtype, Groups p, unsigned gy, unsigned gz, hipStream_t stream) {
  if (dtype != DT_F32 && dtype != DT_BF16) return ERR_BAD_DTYPE;
  if (mfma_fits(dtype, p) && p.tm == TM_SMALL) {
    const dim3 grid((unsigned)((p.N + 15) / 16), gy, gz);
    grouped_mfma_small_kernel<bf16, GATED><<<grid, 256, 0, stream>>>(p);
  } else if (mfma_fits(dtype, p) && p.tm == TM_BIG) {
    const int cols = GATED ? 64 : 128;
    const dim3 grid((unsigned)((p.N + cols - 1) / cols), gy, gz);
    grouped_mfma_big_kernel<bf16, GATED><<<grid, 256, 0, stream>>>(p);
  } else {
    if (p.tm > BM) return ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((p.N + BN - 1) / BN), gy, gz);
    if (dtype == DT_F32) grouped_valu_kernel<float, float, GATED><<<grid, 256, 0, stream>>>(p);
    else grouped_valu_kernel<bf16, bf16, GATED><<<grid, 256, 0, stream>>>(p);
  }
  return launch_status();
}

}  // namespace

// C[m, z*c_zs + n] = (sigmoid(gate[m, z]) *) sum_k A[m, z*a_zs + k] W[z*w_zs + n*ldw + k], z < groups.
extern "C" int dinfer_heads_nt(int dtype, const void* A, int64_t lda, int64_t a_zs, const void* W, int64_t ldw,
                               int64_t w_zs, void* C, int64_t ldc, int64_t c_zs, int64_t M, int64_t N, int64_t K,
                               int64_t groups, const void* gate, int64_t ld_gate, hipStream_t stream) {
  if (M <= 0 || N <= 0 || groups <= 0) return OK;
  if (K <= 0 || ldw < K || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff || groups > 65535) return ERR_BAD_SHAPE;
  Groups p{};
  p.A = A; p.lda = lda; p.a_zs = a_zs; p.W = W; p.ldw = ldw; p.w_zs = w_zs; p.C = C; p.ldc = ldc; p.c_zs = c_zs;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.gate = gate; p.ld_gate = ld_gate;
  p.tm = !mfma_fits(dtype, p) ? BM : M <= TM_SMALL ? TM_SMALL : TM_BIG;
  const int64_t gy = (M + p.tm - 1) / p.tm;
  if (gy > 65535) return ERR_UNSUPPORTED;
  return launch_groups<false>(dtype, p, (unsigned)gy, (unsigned)groups, stream);
}

// The products of the experts (see the head of the file). W [experts][rows][ldw] with w_zs elements an expert;
// gated 1: rows = 2 N (gate rows, then up rows); 0: plain; 2, 3: plain with silu or gelu (error function) on every
// result. max_tiles: the length of `tiles`.
extern "C" int dinfer_experts_nt(int dtype, int gated, const void* A, int64_t lda, const void* W, int64_t ldw,
                                 int64_t w_zs, void* C, int64_t ldc, int64_t N, int64_t K, const int32_t* tiles,
                                 int64_t max_tiles, int tile_rows, const int32_t* offsets, const int32_t* perm, int a_div,
                                 int c_to_perm, hipStream_t stream) {
  if (N <= 0 || max_tiles <= 0) return OK;
  if (K <= 0 || ldw < K || lda < K || ldc < N || N > 0x7fffffff || K > 0x7fffffff || max_tiles > 65535 || !tiles ||
      !offsets || !perm || tile_rows <= 0)
    return ERR_BAD_SHAPE;
  Groups p{};
  p.A = A; p.lda = lda; p.W = W; p.ldw = ldw; p.w_zs = w_zs; p.C = C; p.ldc = ldc;
  p.N = (int)N; p.K = (int)K; p.tiles = tiles; p.offsets = offsets; p.perm = perm; p.a_div = a_div;
  p.c_to_perm = c_to_perm; p.gate_n = (int)N; p.tm = tile_rows;
  if (gated < 0 || gated > 3) return ERR_UNSUPPORTED;
  p.act = gated >= 2 ? gated - 1 : 0;
  if (!mfma_fits(dtype, p) && tile_rows > BM) return ERR_UNSUPPORTED;
  return gated == 1 ? launch_groups<true>(dtype, p, (unsigned)max_tiles, 1, stream)
               : launch_groups<false>(dtype, p, (unsigned)max_tiles, 1, stream);
}

// Rows of a tile for a routed layer's two products: the matrix-core kernels take 16 (few rows an expert: the weights
// are streamed) or 128; anything else (float, sizes that are no multiples of 8) runs on the vector ALUs with 64.
extern "C" int dinfer_moe_tile_rows(int dtype, int64_t entries, int experts, int64_t k_in, int64_t k_mid) {
  if (dtype != DT_BF16 || k_in % 8 || k_mid % 8) return BM;
  return entries <= (int64_t)TM_SMALL * experts ? TM_SMALL : TM_BIG;
}


// z: float scratch [tokens, experts + 1].
extern "C" int dinfer_moe_route(int dtype, const void* x, int64_t ld_x, int64_t tokens, const float* router,
                                const float* shared_gate_w, int experts, int top, int width, float* z, int32_t* idx,
                                float* share, float* shared_gate, int all_scores, const float* correction,
                                hipStream_t stream) {
  // all_scores: softmax over all experts, chosen by score + correction (float [experts] or null), weights the scores
  if (tokens <= 0) return OK;
  if (experts <= 0 || top <= 0 || top > experts || width <= 0 || tokens > 0x7fffffff || !z) return ERR_BAD_SHAPE;
  if (experts > MAX_EXPERTS || top > 64) return ERR_UNSUPPORTED;
  const int rows = experts + (shared_gate_w ? 1 : 0), ldz = experts + 1;
  const int rt = tokens <= 128 ? 1 : 8;
  const dim3 grid((unsigned)((tokens + rt - 1) / rt), (unsigned)((rows + 3) / 4));
  const bool x8 = dtype == DT_BF16 && width % 8 == 0 && ld_x % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
                  ((uintptr_t)router % 16) == 0 && ((uintptr_t)shared_gate_w % 16) == 0;
  if (x8) {
    if (rt == 1)
      moe_logits_bf16x8_kernel<1><<<grid, 256, 0, stream>>>((const bf16*)x, ld_x, (int)tokens, router, shared_gate_w,
                                                            experts, width, z, ldz);
    else
      moe_logits_bf16x8_kernel<8><<<grid, 256, 0, stream>>>((const bf16*)x, ld_x, (int)tokens, router, shared_gate_w,
                                                            experts, width, z, ldz);
  } else
  DINFER_DISPATCH_DTYPE(dtype, {
    if (rt == 1)
      moe_logits_kernel<S, 1><<<grid, 256, 0, stream>>>((const S*)x, ld_x, (int)tokens, router, shared_gate_w, experts,
                                                        width, z, ldz);
    else
      moe_logits_kernel<S, 8><<<grid, 256, 0, stream>>>((const S*)x, ld_x, (int)tokens, router, shared_gate_w, experts,
                                                        width, z, ldz);
  });
  if (launch_status() != OK) return ERR_LAUNCH;
  moe_topk_kernel<<<(unsigned)((tokens + 3) / 4), 256, 0, stream>>>(z, ldz, (int)tokens, experts, top,
                                                                   shared_gate_w ? 1 : 0, idx, share, shared_gate,
                                                                   all_scores, correction);
  return launch_status();
}

extern "C" int dinfer_moe_scatter(const int32_t* idx, int64_t entries, int experts, int tile_rows, int32_t* offsets,
                                  int32_t* perm, int32_t* tiles, int64_t max_tiles, int real_experts,
                                  hipStream_t stream) {
  // real_experts < experts: the experts from there on get no tiles (0 or less: all are real)
  if (real_experts <= 0 || real_experts > experts) real_experts = experts;
  if (entries <= 0) return OK;
  if (experts <= 0 || tile_rows <= 0 || entries > 0x7fffffff ||
      max_tiles < (entries + tile_rows - 1) / tile_rows + experts)
    return ERR_BAD_SHAPE;
  if (experts > MAX_EXPERTS) return ERR_UNSUPPORTED;
  moe_scatter_kernel<<<1, 1024, 0, stream>>>(idx, (int)entries, experts, tile_rows, offsets, perm, tiles, (int)max_tiles,
                                             real_experts);
  return launch_status();
}

extern "C" int dinfer_moe_combine(int dtype, const void* y, int64_t ld_y, const float* share, int top, const void* shared,
                                  int64_t ld_s, const float* shared_gate, void* out, int64_t ld_o, int64_t tokens,
                                  int width, const int32_t* idx, int real_experts, const void* x, int64_t ld_x,
                                  hipStream_t stream) {
  // idx (may be null) [tokens, top] with real_experts: a choice from real_experts on adds its share of x[t], the
  // token's input, instead of a row of y.
  if (tokens <= 0) return OK;
  if (top <= 0 || width <= 0 || tokens > 0x7fffffff || (idx && (!x || ld_x < width))) return ERR_BAD_SHAPE;
  const bool vec = dtype == DT_BF16 && width % 8 == 0 && ld_y % 8 == 0 && ld_o % 8 == 0 && (!shared || ld_s % 8 == 0) &&
                   ((uintptr_t)y % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)shared % 16) == 0 &&
                   (!idx || (ld_x % 8 == 0 && ((uintptr_t)x % 16) == 0));
  if (vec) {
    moe_combine_bf16x8_kernel<<<(unsigned)tokens, width >= 2048 ? 256 : 64, 0, stream>>>(
        (const bf16*)y, ld_y, share, top, (const bf16*)shared, ld_s, shared_gate, (bf16*)out, ld_o, width, idx,
        real_experts, (const bf16*)x, ld_x);
    return launch_status();
  }
  DINFER_DISPATCH_DTYPE(dtype, {
    moe_combine_kernel<S><<<(unsigned)tokens, 256, 0, stream>>>((const S*)y, ld_y, share, top, (const S*)shared, ld_s,
                                                               shared_gate, (S*)out, ld_o, width, idx, real_experts,
                                                               (const S*)x, ld_x);
  });
  return launch_status();
}
