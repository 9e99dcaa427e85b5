// Linear recurrences with a scalar decay: per request and head one matrix S [D, V] in float,
//
//   per token:   S <- a_t S + c_t k_t v_t^T;   o_t = S^T q_t
//
// with a_t in (0, 1] a decay (one a head, or one a head and token) and c_t an optional step size a head and token.
// Two mixers are this recurrence with different things around it:
//
//   retention       q, k rotated by the position, k scaled; a fixed decay a head; no step size
//   state space     q = C_t, k = B_t (shared by the heads of a group), v = x_t; a_t = exp(-exp(A) dt_t), c_t = dt_t;
//                   x, B and C come out of a short causal convolution with bias and silu
//
//   rot_widen          a thread an entry: q and k heads rotated (pairs (i, i + rot/2) of the first rot entries) by the
//                      table row of the token's position, k times a scale, v widened; float out
//   conv_silu          a thread a (token, channel): taps over the step's rows and the request's stored inputs, bias, silu;
//                      the threads behind the channels make dt = softplus(. + bias) and exp(-exp(A) dt) of every head
//   decay_recurrence   token by token, one request, one head and 8 columns of S a workgroup: the 32 lanes of half a wave
//                      share a column and own a strip of its rows; 16 tokens' operands wait in LDS while the next 16 are
//                      on their way in registers. Serves single decoded rows (the whole state in and out once) and
//                      prompt portions of any length
//   gated_group_norm   (y + skip_h x) * silu(z), then divided by the root mean square of its group of columns, times a
//                      gain a column; or the gate after the norm; one workgroup a (token, group)
//
// S is stored transposed, [slot][head][V][D], as the delta rule's state is: a thread's strip is contiguous.
// A request whose step starts at position 0 starts from S = 0 and zero stored inputs, whatever its slot held.
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int CH = 16;          // tokens of a chunk in the token-by-token recurrence
constexpr int COLS = 8;         // columns of S a workgroup
constexpr int MAX_TAPS = 16;

__device__ __forceinline__ int request_of(const int32_t* __restrict__ cu, int num_reqs, int t) {
  int lo = 0, hi = num_reqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// work row: q (H D) | k (H D) | v (H V), float; a thread an entry
template <class S>
__global__ void __launch_bounds__(256) rot_widen_kernel(const S* __restrict__ proj, int64_t ld, int64_t q_off,
                                                        int64_t k_off, int64_t v_off, const int32_t* __restrict__ pos,
                                                        const float* __restrict__ cos_sin, int rot, float k_scale,
                                                        float* __restrict__ work, int64_t ldw, int H, int D, int V) {
  const int64_t t = blockIdx.x;
  const S* row = proj + t * ld;
  float* wr = work + t * ldw;
  const int half = rot / 2;
  const int hd = H * D;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= 2 * hd + H * V) return;
  if (c >= 2 * hd) {
    wr[c] = to_f32(row[v_off + c - 2 * hd]);
    return;
  }
  const bool is_k = c >= hd;
  const int e = is_k ? c - hd : c;
  const int d = e % D;
  const S* src = row + (is_k ? k_off : q_off);
  float y = to_f32(src[e]);
  if (cos_sin && d < rot) {
    const float* cs = cos_sin + (int64_t)pos[t] * rot;
    const bool first = d < half;
    const int i = first ? d : d - half;
    const float other = to_f32(src[first ? e + half : e - half]);
    y = first ? rotated_first(y, other, cs[i], cs[half + i]) : rotated_second(other, y, cs[i], cs[half + i]);
  }
  wr[c] = is_k ? y * k_scale : y;
}

// The same for bfloat16 rows whose sizes are multiples of 8 (half the rotated entries too): a thread takes 8 consecutive
// entries of a head, so they lie wholly in the first half of the rotated entries, in the second, or behind them; its
// values, its partners' and the angles come as 16- and 32-byte loads and the floats leave as two 16-byte stores.
__global__ void __launch_bounds__(256) rot_widen_vec_kernel(const bf16* __restrict__ proj, int64_t ld, int64_t q_off,
                                                            int64_t k_off, int64_t v_off, const int32_t* __restrict__ pos,
                                                            const float* __restrict__ cos_sin, int rot, float k_scale,
                                                            float* __restrict__ work, int64_t ldw, int H, int D, int V) {
  const int64_t t = blockIdx.x;
  const bf16* row = proj + t * ld;
  float* wr = work + t * ldw;
  const int half = rot / 2;
  const int hd = H * D;
  const int c = 8 * (blockIdx.y * 256 + threadIdx.x);
  if (c >= 2 * hd + H * V) return;
  float y[8];
  if (c >= 2 * hd) {
    const bf16x8 v = *(const bf16x8*)(row + v_off + c - 2 * hd);
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (float)v[e];
  } else {
    const bool is_k = c >= hd;
    const int e0 = is_k ? c - hd : c;
    const int d = e0 % D;
    const bf16* src = row + (is_k ? k_off : q_off);
    const bf16x8 v = *(const bf16x8*)(src + e0);
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (float)v[e];
    if (cos_sin && d < rot) {
      const float* cs = cos_sin + (int64_t)pos[t] * rot;
      const bool first = d < half;
      const int i = first ? d : d - half;
      const bf16x8 o = *(const bf16x8*)(src + (first ? e0 + half : e0 - half));
      const f32x4 c0 = *(const f32x4*)(cs + i), c1 = *(const f32x4*)(cs + i + 4);
      const f32x4 s0 = *(const f32x4*)(cs + half + i), s1 = *(const f32x4*)(cs + half + i + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float cc = e < 4 ? c0[e & 3] : c1[e & 3], sn = e < 4 ? s0[e & 3] : s1[e & 3];
        const float other = (float)o[e];
        y[e] = first ? rotated_first(y[e], other, cc, sn) : rotated_second(other, y[e], cc, sn);
      }
    }
    if (is_k) {
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] *= k_scale;
    }
  }
  f32x4 a, b;
#pragma unroll
  for (int e = 0; e < 4; ++e) { a[e] = y[e]; b[e] = y[4 + e]; }
  *(f32x4*)(wr + c) = a;
  *(f32x4*)(wr + c + 4) = b;
}

// work row: the C channels after convolution, bias and silu | dt (H) | decay (H), float
template <class S>
__global__ void __launch_bounds__(256) conv_silu_kernel(
    const S* __restrict__ proj, int64_t ld, int64_t x_off, int64_t dt_off, const float* __restrict__ taps,
    const float* __restrict__ bias, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const S* __restrict__ conv_state, const int32_t* __restrict__ slots, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ seq_lens, float* __restrict__ work, int64_t ldw, int num_reqs, int C, int H, int K) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C + H) return;
  const S* row = proj + (int64_t)t * ld;
  float* wr = work + (int64_t)t * ldw;
  if (c >= C) {
    const int h = c - C;
    const float dt = softplus_f(to_f32(row[dt_off + h]) + dt_bias[h]);
    wr[C + h] = dt;
    wr[C + H + h] = expf(-expf(a_log[h]) * dt);
    return;
  }
  const int b = request_of(cu, num_reqs, t);
  const int i = t - cu[b];                                   // index of the token in its request's rows of this step
  const int start = seq_lens[b] - (cu[b + 1] - cu[b]);       // position of the request's first row of this step
  const S* old = (K > 1 && start > 0) ? conv_state + (int64_t)slots[b] * C * (K - 1) : nullptr;
  float acc = bias ? bias[c] : 0.f;
  for (int j = K - 1; j >= 0; --j) {                         // the oldest input first
    float x = 0.f;
    if (i - j >= 0) x = to_f32(row[x_off + c - (int64_t)j * ld]);
    else if (old) x = to_f32(old[(int64_t)c * (K - 1) + (K - 1 + i - j)]);
    acc = __builtin_fmaf(taps[(int64_t)c * K + (K - 1 - j)], x, acc);
  }
  wr[c] = silu_f(acc);
}

// The same for bfloat16 rows and K taps known when compiled: a thread takes 8 consecutive channels of a token, so a
// row's inputs come as one 16-byte load a tap (the K rows are asked for before the first is used), the 8 K taps of
// its channels are consecutive floats, and the result leaves as two 16-byte stores. The stored inputs of a request
// ([channel][K - 1]) are read one value at a time: only the first K - 1 rows of a request's portion need them.
template <int K>
__global__ void __launch_bounds__(256) conv_silu_vec_kernel(
    const bf16* __restrict__ proj, int64_t ld, int64_t x_off, int64_t dt_off, const float* __restrict__ taps,
    const float* __restrict__ bias, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const bf16* __restrict__ conv_state, const int32_t* __restrict__ slots, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ seq_lens, float* __restrict__ work, int64_t ldw, int num_reqs, int C, int H) {
  const int t = blockIdx.x;
  const int u = blockIdx.y * 256 + threadIdx.x;
  const int pieces = C / 8;
  if (u >= pieces + H) return;
  const bf16* row = proj + (int64_t)t * ld;
  float* wr = work + (int64_t)t * ldw;
  if (u >= pieces) {
    const int h = u - pieces;
    const float dt = softplus_f((float)row[dt_off + h] + dt_bias[h]);
    wr[C + h] = dt;
    wr[C + H + h] = expf(-expf(a_log[h]) * dt);
    return;
  }
  const int c = 8 * u;
  const int b = request_of(cu, num_reqs, t);
  const int i = t - cu[b];
  const int start = seq_lens[b] - (cu[b + 1] - cu[b]);
  const bf16* old = (K > 1 && start > 0) ? conv_state + (int64_t)slots[b] * C * (K - 1) : nullptr;
  bf16x8 in[K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    if (i - j >= 0) {
      in[j] = *(const bf16x8*)(row + x_off + c - (int64_t)j * ld);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        in[j][e] = old ? old[(int64_t)(c + e) * (K - 1) + (K - 1 + i - j)] : (bf16)0.f;
    }
  }
  float tap[8 * K];
#pragma unroll
  for (int e = 0; e < 2 * K; ++e) {
    const f32x4 w = *(const f32x4*)(taps + (int64_t)c * K + 4 * e);
    tap[4 * e] = w[0]; tap[4 * e + 1] = w[1]; tap[4 * e + 2] = w[2]; tap[4 * e + 3] = w[3];
  }
  float acc[8];
  if (bias) {
    const f32x4 b0 = *(const f32x4*)(bias + c), b1 = *(const f32x4*)(bias + c + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { acc[e] = b0[e]; acc[4 + e] = b1[e]; }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  }
#pragma unroll
  for (int j = K - 1; j >= 0; --j)                           // the oldest input first, as the kernel above
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(tap[e * K + (K - 1 - j)], (float)in[j][e], acc[e]);
  f32x4 o0, o1;
#pragma unroll
  for (int e = 0; e < 4; ++e) { o0[e] = silu_f(acc[e]); o1[e] = silu_f(acc[4 + e]); }
  *(f32x4*)(wr + c) = o0;
  *(f32x4*)(wr + c + 4) = o1;
}

// A lane's value plus that of the lane a DPP pattern pairs it with (full-rate vector instructions, no LDS).
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// The sum over 32 lanes (two DPP rows of 16), in every lane of them.
__device__ __forceinline__ float half_wave_sum(float v) {
  v = dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  v = dpp_add<0x141>(v);   // row_half_mirror
  v = dpp_add<0x140>(v);   // row_mirror
  return v + __shfl_xor(v, 16, WAVE);
}

struct Operands {
  const float* q; int64_t ldq;        // [T, G D]
  const float* k; int64_t ldk;        // [T, G D]
  const float* v; int64_t ldv;        // [T, H V]
  const float* decay; int64_t ldd;    // [T, H], or [H] with ldd = 0
  const float* gain; int64_t ldg;     // [T, H] or null
};

// One request, one head and COLS columns of S a workgroup; a thread owns RPT consecutive rows of a column (D <= 32 RPT).
template <int RPT>
__global__ void __launch_bounds__(256) decay_recurrence_kernel(Operands p, float* __restrict__ state,
                                                               const int32_t* __restrict__ slots,
                                                               const int32_t* __restrict__ cu,
                                                               const int32_t* __restrict__ seq_lens,
                                                               float* __restrict__ out, int64_t ld_out, int G, int H,
                                                               int D, int V) {
  constexpr int DP = 32 * RPT;
  __shared__ __attribute__((aligned(16))) float ks[CH][DP];
  __shared__ __attribute__((aligned(16))) float qs[CH][DP];
  __shared__ float vs[CH][COLS];
  __shared__ float as[CH];
  // the request is the slowest index of the grid: the workgroups of one long request among many short ones then
  // spread over all XCDs (consecutive workgroups go to consecutive XCDs) instead of meeting on one
  const int b = blockIdx.z, h = blockIdx.y, cb = blockIdx.x;
  const int tid = threadIdx.x;
  const int rg = tid & 31, cj = tid >> 5;
  const int j = cb * COLS + cj;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  const int start = seq_lens[b] - n;
  const int g = h / (H / G);
  const bool col_ok = j < V;
  float* sp = state + ((((int64_t)slots[b] * H + h) * V + (col_ok ? j : 0)) * D) + rg * RPT;
  float S[RPT];
  // a strip of a multiple of 4 rows in a matrix of a multiple of 4 rows moves 16 bytes at a time
  const bool quads = RPT % 4 == 0 && D % 4 == 0;
  if (quads) {
#pragma unroll
    for (int i = 0; i < RPT; i += 4) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (start > 0 && col_ok && rg * RPT + i < D) v = *(const f32x4*)(sp + i);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i + e < RPT) S[i + e] = v[e];
    }
  } else {
#pragma unroll
    for (int i = 0; i < RPT; ++i) S[i] = (start > 0 && col_ok && rg * RPT + i < D) ? sp[i] : 0.f;
  }

  // what a thread carries of the next chunk: entries of k and of q, one of v (times its step size), one decay
  constexpr int PK = (CH * DP) / 256;
  float pk[PK], pq[PK], pv = 0.f, pa = 0.f;
  auto fetch = [&](int ct) {
#pragma unroll
    for (int e = 0; e < PK; ++e) {
      const int idx = tid + e * 256;
      const int tok = idx / DP, d = idx % DP;
      const bool ok = ct + tok < n && d < D;
      const int64_t t = t0 + ct + tok;
      pk[e] = ok ? p.k[t * p.ldk + g * D + d] : 0.f;
      pq[e] = ok ? p.q[t * p.ldq + g * D + d] : 0.f;
    }
    if (tid < CH * COLS) {
      const int tok = tid / COLS, c = tid % COLS;
      const int col = cb * COLS + c;
      const int64_t t = t0 + ct + tok;
      pv = 0.f;
      if (ct + tok < n && col < V) {
        pv = p.v[t * p.ldv + h * V + col];
        if (p.gain) pv *= p.gain[t * p.ldg + h];
      }
    }
    if (tid < CH) pa = ct + tid < n ? p.decay[(int64_t)(t0 + ct + tid) * p.ldd + h] : 1.f;
  };
  fetch(0);
  for (int ct = 0; ct < n; ct += CH) {
    __syncthreads();  // the chunk before has been consumed
#pragma unroll
    for (int e = 0; e < PK; ++e) {
      const int idx = tid + e * 256;
      ks[idx / DP][idx % DP] = pk[e];
      qs[idx / DP][idx % DP] = pq[e];
    }
    if (tid < CH * COLS) vs[tid / COLS][tid % COLS] = pv;
    if (tid < CH) as[tid] = pa;
    __syncthreads();
    if (ct + CH < n) fetch(ct + CH);  // in flight while this chunk is worked through
    const int m = n - ct < CH ? n - ct : CH;
    // four tokens a round: only the state's update runs from token to token, the four row sums meet the lanes
    // together; what is left of the step's rows (all of a single decoded row) goes token by token
    int t4 = 0;
    for (; t4 + 4 <= m; t4 += 4) {
      float part[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int tok = t4 + u;
        const float a = as[tok], vt = vs[tok][cj];
        float o0 = 0.f, o1 = 0.f;   // two chains: a fixed order all the same
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
          S[i] = __builtin_fmaf(ks[tok][rg * RPT + i], vt, a * S[i]);
          if (i & 1) o1 = __builtin_fmaf(S[i], qs[tok][rg * RPT + i], o1);
          else o0 = __builtin_fmaf(S[i], qs[tok][rg * RPT + i], o0);
        }
        part[u] = o0 + o1;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) part[u] = half_wave_sum(part[u]);
      if (rg < 4 && col_ok) {
        const float o = rg == 0 ? part[0] : rg == 1 ? part[1] : rg == 2 ? part[2] : part[3];
        out[(int64_t)(t0 + ct + t4 + rg) * ld_out + h * V + j] = o;
      }
    }
    for (int tok = t4; tok < m; ++tok) {
      const float a = as[tok], vt = vs[tok][cj];
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        S[i] = __builtin_fmaf(ks[tok][rg * RPT + i], vt, a * S[i]);
        if (i & 1) o1 = __builtin_fmaf(S[i], qs[tok][rg * RPT + i], o1);
        else o0 = __builtin_fmaf(S[i], qs[tok][rg * RPT + i], o0);
      }
      const float o = half_wave_sum(o0 + o1);
      if (rg == 0 && col_ok) out[(int64_t)(t0 + ct + tok) * ld_out + h * V + j] = o;
    }
  }
  if (col_ok && quads) {
#pragma unroll
    for (int i = 0; i < RPT; i += 4) {
      f32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = S[i + e < RPT ? i + e : 0];
      if (rg * RPT + i < D) *(f32x4*)(sp + i) = v;
    }
  } else if (col_ok) {
#pragma unroll
    for (int i = 0; i < RPT; ++i)
      if (rg * RPT + i < D) sp[i] = S[i];
  }
}

// gate_first: out[t, col_off + c] = u / sqrt(mean over c's group of u^2 + eps) * w[c],  u = (y[t, c] + skip[c / V] x[t, c]) * silu(z[t, c]);
// else the gate comes after the norm: u = y + skip x, out = u / sqrt(mean u^2 + eps) * w[c] * silu(z[t, c])
template <class S>
__global__ void __launch_bounds__(256) gated_group_norm_kernel(const float* __restrict__ y, int64_t ld_y,
                                                               const float* __restrict__ x, int64_t ld_x,
                                                               const float* __restrict__ skip, int V,
                                                               const S* __restrict__ z, int64_t ld_z, int64_t z_off,
                                                               const float* __restrict__ w, S* __restrict__ out,
                                                               int64_t ld_out, int64_t col_off, int group, float eps,
                                                               float out_scale, int gate_first) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int c0 = blockIdx.y * group;
  auto value = [&](int c) {
    float u = y[t * ld_y + c];
    if (skip) u = __builtin_fmaf(skip[c / V], x[t * ld_x + c], u);
    return gate_first ? u * silu_f(to_f32(z[t * ld_z + z_off + c])) : u;
  };
  float ss = 0.f;
  constexpr int KEEP = 4;                    // a group of up to 1,024 columns stays in registers between the two passes
  float kept[KEEP];
  const bool keeps = group <= 256 * KEEP;
#pragma unroll
  for (int e = 0; e < KEEP; ++e) {
    const int c = c0 + threadIdx.x + 256 * e;
    kept[e] = (keeps && c < c0 + group) ? value(c) : 0.f;
    ss = __builtin_fmaf(kept[e], kept[e], ss);
  }
  if (!keeps)
    for (int c = c0 + threadIdx.x; c < c0 + group; c += 256) {
      const float u = value(c);
      ss = __builtin_fmaf(u, u, ss);
    }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)group + eps);
  if (keeps) {
#pragma unroll
    for (int e = 0; e < KEEP; ++e) {
      const int c = c0 + threadIdx.x + 256 * e;
      if (c < c0 + group) {
        float r = kept[e] * inv * (w ? w[c] : 1.f) * out_scale;
        if (!gate_first) r *= silu_f(to_f32(z[t * ld_z + z_off + c]));
        out[t * ld_out + col_off + c] = from_f32<S>(r);
      }
    }
    return;
  }
  for (int c = c0 + threadIdx.x; c < c0 + group; c += 256) {
    float r = value(c) * inv * (w ? w[c] : 1.f) * out_scale;
    if (!gate_first) r *= silu_f(to_f32(z[t * ld_z + z_off + c]));
    out[t * ld_out + col_off + c] = from_f32<S>(r);
  }
}

// The same for groups of up to 256 columns: a wave a (token, group), a lane up to 4 of its columns, the sum of squares by
// shuffles; no LDS and no barrier (a retention's groups are its heads: 128 columns were half a workgroup idle).
template <class S>
__global__ void __launch_bounds__(256) gated_group_norm_wave_kernel(const float* __restrict__ y, int64_t ld_y,
                                                                    const float* __restrict__ x, int64_t ld_x,
                                                                    const float* __restrict__ skip, int V,
                                                                    const S* __restrict__ z, int64_t ld_z, int64_t z_off,
                                                                    const float* __restrict__ w, S* __restrict__ out,
                                                                    int64_t ld_out, int64_t col_off, int groups, int group,
                                                                    float eps, float out_scale, int gate_first) {
  const int64_t t = blockIdx.x;
  const int g = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (g >= groups) return;                   // (a whole wave leaves: the shuffles below see full waves only)
  const int c0 = g * group;
  float kept[4], gate[4];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int i = lane + 64 * e;
    kept[e] = 0.f;
    gate[e] = 0.f;
    if (i < group) {
      const int c = c0 + i;
      float u = y[t * ld_y + c];
      if (skip) u = __builtin_fmaf(skip[c / V], x[t * ld_x + c], u);
      gate[e] = silu_f(to_f32(z[t * ld_z + z_off + c]));
      kept[e] = gate_first ? u * gate[e] : u;
    }
    ss = __builtin_fmaf(kept[e], kept[e], ss);
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)group + eps);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int i = lane + 64 * e;
    if (i < group) {
      const int c = c0 + i;
      float r = kept[e] * inv * (w ? w[c] : 1.f) * out_scale;
      if (!gate_first) r *= gate[e];
      out[t * ld_out + col_off + c] = from_f32<S>(r);
    }
  }
}

}  // namespace

// proj [T, ld] in the step's dtype: H heads of q (size D) from column q_off, of k from k_off, H heads of v (size V) from
// v_off. cos_sin float [positions, rot] = [cos | sin] (null or rot 0: no rotation). work [T, ldw] float:
// q (H D) | k (H D) | v (H V), k times k_scale.
extern "C" int dinfer_rot_widen(int dtype, const void* proj, int64_t ld, int64_t q_off, int64_t k_off, int64_t v_off,
                                const int32_t* positions, const float* cos_sin, int rot, float k_scale, float* work,
                                int64_t ldw, int64_t tokens, int H, int D, int V, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (H <= 0 || D <= 0 || V <= 0 || rot < 0 || rot > D || rot % 2 || tokens > 0x7fffffff ||
      ldw < 2 * (int64_t)H * D + (int64_t)H * V)
    return ERR_BAD_SHAPE;
  const bool vec = dtype == DT_BF16 && D % 8 == 0 && V % 8 == 0 && (!cos_sin || rot % 16 == 0) && ld % 8 == 0 &&
                   q_off % 8 == 0 && k_off % 8 == 0 && v_off % 8 == 0 && ldw % 4 == 0 && ((uintptr_t)proj % 16) == 0 &&
                   ((uintptr_t)work % 16) == 0 && ((uintptr_t)cos_sin % 16) == 0;
  if (vec) {
    const int pieces = (2 * H * D + H * V) / 8;
    const dim3 vgrid((unsigned)tokens, (unsigned)((pieces + 255) / 256));
    rot_widen_vec_kernel<<<vgrid, 256, 0, stream>>>((const bf16*)proj, ld, q_off, k_off, v_off, positions, cos_sin, rot,
                                                    k_scale, work, ldw, H, D, V);
    return launch_status();
  }
  const dim3 grid((unsigned)tokens, (unsigned)((2 * H * D + H * V + 255) / 256));
  DINFER_DISPATCH_DTYPE(dtype, {
    rot_widen_kernel<S><<<grid, 256, 0, stream>>>((const S*)proj, ld, q_off, k_off, v_off, positions, cos_sin,
                                                              rot, k_scale, work, ldw, H, D, V);
  });
  return launch_status();
}

// proj [T, ld]: C channels from column x_off (they pass the convolution), H step-size logits from dt_off. taps [C, K]
// float, the last column the current token's; bias [C] float or null; a_log, dt_bias [H] float. conv_state
// [slots, C, K - 1] in the step's dtype (unused with K = 1). work [T, ldw] float, ldw >= C + 2 H.
extern "C" int dinfer_conv_silu(int dtype, const void* proj, int64_t ld, int64_t x_off, int64_t dt_off, const float* taps,
                                const float* bias, const float* a_log, const float* dt_bias, const void* conv_state,
                                const int32_t* state_slots, const int32_t* cu_seqlens, const int32_t* seq_lens,
                                float* work, int64_t ldw, int num_reqs, int64_t tokens, int C, int H, int K,
                                hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (C <= 0 || H <= 0 || K <= 0 || tokens > 0x7fffffff || ldw < (int64_t)C + 2 * H) return ERR_BAD_SHAPE;
  if (K > MAX_TAPS) return ERR_UNSUPPORTED;
  // (single decoded rows take all their earlier inputs from the stored ones, a value at a time: the kernel of a thread
  // a channel is the faster one there; both add in the same order and give the same bits)
  const bool vec = tokens >= 4 * (int64_t)num_reqs && dtype == DT_BF16 && K >= 2 && K <= 4 && C % 8 == 0 && ld % 8 == 0 && x_off % 8 == 0 && ldw % 4 == 0 &&
                   ((uintptr_t)proj % 16) == 0 && ((uintptr_t)work % 16) == 0 && ((uintptr_t)taps % 16) == 0 &&
                   ((uintptr_t)bias % 16) == 0;
  if (vec) {
    const dim3 vgrid((unsigned)tokens, (unsigned)((C / 8 + H + 255) / 256));
#define DINFER_CONV_VEC(K_)                                                                                          \
  conv_silu_vec_kernel<K_><<<vgrid, 256, 0, stream>>>((const bf16*)proj, ld, x_off, dt_off, taps, bias, a_log, dt_bias, \
                                                      (const bf16*)conv_state, state_slots, cu_seqlens, seq_lens, work, \
                                                      ldw, num_reqs, C, H)
    if (K == 2) DINFER_CONV_VEC(2);
    else if (K == 3) DINFER_CONV_VEC(3);
    else DINFER_CONV_VEC(4);
#undef DINFER_CONV_VEC
    return launch_status();
  }
  const dim3 grid((unsigned)tokens, (unsigned)((C + H + 255) / 256));
  DINFER_DISPATCH_DTYPE(dtype, {
    conv_silu_kernel<S><<<grid, 256, 0, stream>>>((const S*)proj, ld, x_off, dt_off, taps, bias, a_log, dt_bias,
                                                  (const S*)conv_state, state_slots, cu_seqlens, seq_lens, work, ldw,
                                                  num_reqs, C, H, K);
  });
  return launch_status();
}

// q, k [T, G D], v [T, H V] float; decay [T, H] (ld_decay its row stride) or [H] (ld_decay 0); gain [T, H] or null.
// state [slots, H, V, D] float (S transposed); out [T, ld_out] float, head h at column h V.
extern "C" int dinfer_decay_recurrence(const float* q, int64_t ldq, const float* k, int64_t ldk, const float* v,
                                       int64_t ldv, const float* decay, int64_t ld_decay, const float* gain,
                                       int64_t ld_gain, float* state, const int32_t* state_slots,
                                       const int32_t* cu_seqlens, const int32_t* seq_lens, float* out, int64_t ld_out,
                                       int num_reqs, int G, int H, int D, int V, hipStream_t stream) {
  if (num_reqs <= 0) return OK;
  if (G <= 0 || H <= 0 || H % G || D <= 0 || V <= 0 || num_reqs > 65535 || H > 65535 || !decay) return ERR_BAD_SHAPE;
  if (D > 256) return ERR_UNSUPPORTED;
  Operands p{q, ldq, k, ldk, v, ldv, decay, ld_decay, gain, ld_gain};
  const dim3 grid((unsigned)((V + COLS - 1) / COLS), (unsigned)H, (unsigned)num_reqs);
#define DECAY_REC(R_) \
  decay_recurrence_kernel<R_><<<grid, 256, 0, stream>>>(p, state, state_slots, cu_seqlens, seq_lens, out, ld_out, G, H, D, V)
  if (D <= 32) DECAY_REC(1);
  else if (D <= 64) DECAY_REC(2);
  else if (D <= 128) DECAY_REC(4);
  else DECAY_REC(8);
#undef DECAY_REC
  return launch_status();
}

// y [T, ld_y] float, `groups` groups of `group` columns each; x [T, ld_x] float with skip [groups * group / V] (both or
// neither); z [T, ld_z] in the step's dtype, the gate's columns from z_off; w [groups * group] float or null.
extern "C" int dinfer_gated_group_norm(int dtype, const float* y, int64_t ld_y, const float* x, int64_t ld_x,
                                       const float* skip, int V, const void* z, int64_t ld_z, int64_t z_off,
                                       const float* w, void* out, int64_t ld_out, int64_t col_off, int64_t tokens,
                                       int groups, int group, float eps, float out_scale, int gate_first,
                                       hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (groups <= 0 || group <= 0 || groups > 65535 || tokens > 0x7fffffff || (skip && (!x || V <= 0))) return ERR_BAD_SHAPE;
  if (group <= 256) {
    const dim3 wgrid((unsigned)tokens, (unsigned)((groups + 3) / 4));
    DINFER_DISPATCH_DTYPE(dtype, {
      gated_group_norm_wave_kernel<S><<<wgrid, 256, 0, stream>>>(y, ld_y, x, ld_x, skip, V, (const S*)z, ld_z, z_off, w,
                                                                (S*)out, ld_out, col_off, groups, group, eps, out_scale,
                                                                gate_first);
    });
    return launch_status();
  }
  const dim3 grid((unsigned)tokens, (unsigned)groups);
  DINFER_DISPATCH_DTYPE(dtype, {
    gated_group_norm_kernel<S><<<grid, 256, 0, stream>>>(y, ld_y, x, ld_x, skip, V, (const S*)z, ld_z, z_off, w, (S*)out,
                                                         ld_out, col_off, group, eps, out_scale, gate_first);
  });
  return launch_status();
}
