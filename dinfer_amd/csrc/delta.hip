// Gated delta rule: a recurrent mixer whose state is one matrix S [D, V] a head and request, in float.
//
//   per token, per head:   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
//
// with q and k unit vectors (q times q_scale), g in (0, 1) a decay and beta in (0, 1) a step size, all float. q, k and
// v come out of a short causal convolution over time (a few taps a channel) and silu; the convolution's last
// taps - 1 inputs are state as well. Four kernels serve prompt portions and single decoded rows alike:
//
//   delta_prep         one wave a (token, head of q, k or v): convolution over the step's rows and the request's
//                      stored inputs, silu, unit norm of q and k; one more wave a token makes beta and g. Float out.
//   delta_recurrence   the recurrence, token by token, for one request, one head and 8 columns of S a workgroup.
//                      A thread owns a strip of rows of one column: the 32 lanes of half a wave share a column and
//                      meet once a token, by four DPP additions and one exchange for each of three sums. k, q, v, beta and g of 16
//                      tokens wait in LDS while the next 16 are on their way in registers.
//   delta_conv_update  moves the step's last taps - 1 inputs into the request's stored inputs (after prep has read
//                      the old ones).
//   delta_out          o / rms(o) * w * silu(gate) per head, one wave a (token, head), rounded once on store.
//
// S is stored transposed, [slot][head][V][D]: a thread's strip is contiguous, a wave reads and writes 2 KB to 8 KB in
// one piece, which is what a decode step (one token a request: all of S in and out) is made of.
// A request whose step starts at position 0 starts from S = 0 and zero stored inputs, whatever its slot held.
// Nothing depends on how a request's tokens were cut into steps: every token does the same arithmetic in the same order.
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int WAVES = 4;
constexpr int MAX_HEAD = 512;   // the largest D or V of the prep and out kernels (8 values a lane)
constexpr int MAX_TAPS = 16;
constexpr int CH = 16;          // tokens of a chunk in the recurrence
constexpr int COLS = 8;         // columns of S a workgroup

__device__ __forceinline__ int request_of(const int32_t* __restrict__ cu, int num_reqs, int t) {
  int lo = 0, hi = num_reqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// work [T, ldw] float: q (G D) | k (G D) | v (H V) | beta (H) | g (H)
template <class S>
__global__ void __launch_bounds__(WAVES * 64) delta_prep_kernel(
    const S* __restrict__ proj, int64_t ld, int64_t qkv_off, int64_t b_off, int64_t a_off,
    const float* __restrict__ taps, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const S* __restrict__ conv_state, const int32_t* __restrict__ slots, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ seq_lens, float* __restrict__ work, int64_t ldw, int num_reqs, int G, int H, int D,
    int V, int K, float eps, float q_scale) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int item = blockIdx.y * WAVES + wave;
  const int items = 2 * G + H + 1;
  if (item >= items) return;
  const int b = request_of(cu, num_reqs, t);
  const int i = t - cu[b];                                   // index of the token in its request's rows of this step
  const int start = seq_lens[b] - (cu[b + 1] - cu[b]);       // position of the request's first row of this step
  const S* row = proj + (int64_t)t * ld;
  float* wr = work + (int64_t)t * ldw;
  const int gd = 2 * G * D;
  if (item == items - 1) {                                   // the step size and the decay of every head
    for (int h = lane; h < H; h += 64) {
      wr[gd + H * V + h] = sigmoid_f(to_f32(row[b_off + h]));
      const float sp = softplus_f(to_f32(row[a_off + h]) + dt_bias[h]);
      wr[gd + H * V + H + h] = expf(-expf(a_log[h]) * sp);
    }
    return;
  }
  const bool qk = item < 2 * G;
  const int c0 = qk ? item * D : gd + (item - 2 * G) * V;   // first channel of the head
  const int n = qk ? D : V;
  const S* old = (K > 1 && start > 0) ? conv_state + (int64_t)slots[b] * (gd + H * V) * (K - 1) : nullptr;
  constexpr int PER = MAX_HEAD / 64;
  float y[PER];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int d = lane + 64 * e;
    y[e] = 0.f;
    if (d < n) {
      const int c = c0 + d;
      float acc = 0.f;
      for (int j = K - 1; j >= 0; --j) {                     // the oldest input first
        float x = 0.f;
        if (i - j >= 0) x = to_f32(row[qkv_off + c - (int64_t)j * ld]);
        else if (old) x = to_f32(old[(int64_t)c * (K - 1) + (K - 1 + i - j)]);
        acc = __builtin_fmaf(taps[(int64_t)c * K + (K - 1 - j)], x, acc);
      }
      y[e] = silu_f(acc);
      ss = __builtin_fmaf(y[e], y[e], ss);
    }
  }
  float mul = 1.f;
  if (qk) {
    ss = wave_sum(ss);
    mul = (item < G ? q_scale : 1.f) / sqrtf(ss + eps);
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int d = lane + 64 * e;
    if (d < n) wr[c0 + d] = y[e] * mul;
  }
}

// The same for head sizes that fill lanes evenly (D / 8 a power of two from 4 to 64 lanes, V a multiple of 8): a lane
// takes 8 consecutive channels of a head (16-byte loads of the step's rows, the taps from a table transposed to
// [K][channels]), the D / 8 lanes of a q or k head meet by shuffles for the unit norm, and a lane stores 32 bytes.
// Lanes beyond the channels make beta and g. One workgroup covers 2,048 channels of a token.
template <class S>
__global__ void __launch_bounds__(256) delta_prep_vec_kernel(
    const S* __restrict__ proj, int64_t ld, int64_t qkv_off, int64_t b_off, int64_t a_off,
    const float* __restrict__ taps_t, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const S* __restrict__ conv_state, const int32_t* __restrict__ slots, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ seq_lens, float* __restrict__ work, int64_t ldw, int num_reqs, int G, int H, int D,
    int V, int K, float eps, float q_scale) {
  const int t = blockIdx.x;
  const int gd = 2 * G * D, C = gd + H * V;
  const int piece = blockIdx.y * 256 + threadIdx.x;   // which 8 channels
  const int b = request_of(cu, num_reqs, t);
  const int i = t - cu[b];
  const int start = seq_lens[b] - (cu[b + 1] - cu[b]);
  const S* row = proj + (int64_t)t * ld;
  float* wr = work + (int64_t)t * ldw;
  const int c = piece * 8;
  if (c >= C) {   // the lanes behind the channels: step sizes and decays
    const int h = c / 8 - C / 8;
    if (h < H) {
      wr[C + h] = sigmoid_f(to_f32(row[b_off + h]));
      const float sp = softplus_f(to_f32(row[a_off + h]) + dt_bias[h]);
      wr[C + H + h] = expf(-expf(a_log[h]) * sp);
    }
    return;
  }
  const S* old = (K > 1 && start > 0) ? conv_state + (int64_t)slots[b] * C * (K - 1) : nullptr;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int j = K - 1; j >= 0; --j) {   // the oldest input first
    float x[8];
    if (i - j >= 0) {
      const S* p = row + qkv_off + c - (int64_t)j * ld;
      if constexpr (sizeof(S) == 2) {
        const bf16x8 v = *(const bf16x8*)p;
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = to_f32(p[e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = old ? to_f32(old[(int64_t)(c + e) * (K - 1) + (K - 1 + i - j)]) : 0.f;
    }
    const float* tp = taps_t + (int64_t)(K - 1 - j) * C + c;
    const f32x4 w0 = *(const f32x4*)tp, w1 = *(const f32x4*)(tp + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(e < 4 ? w0[e] : w1[e - 4], x[e], acc[e]);
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    acc[e] = silu_f(acc[e]);
    ss = __builtin_fmaf(acc[e], acc[e], ss);
  }
  float mul = 1.f;
  if (c < gd) {   // a q or k head: D / 8 neighbouring lanes, aligned to their count
    for (int o = D / 16; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);
    mul = (c < G * D ? q_scale : 1.f) / sqrtf(ss + eps);
  }
  f32x4 o0, o1;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o0[e] = acc[e] * mul;
    o1[e] = acc[4 + e] * mul;
  }
  *(f32x4*)(wr + c) = o0;
  *(f32x4*)(wr + c + 4) = o1;
}

template <class S>
__global__ void __launch_bounds__(256) delta_conv_update_kernel(const S* __restrict__ proj, int64_t ld, int64_t qkv_off,
                                                                S* __restrict__ conv_state,
                                                                const int32_t* __restrict__ slots,
                                                                const int32_t* __restrict__ cu,
                                                                const int32_t* __restrict__ seq_lens, int C, int K) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  const int start = seq_lens[b] - n;
  S* st = conv_state + ((int64_t)slots[b] * C + c) * (K - 1);
  // entry s holds the input of row n - (K - 1) + s of this step; rows before the step come from the old entries,
  // which lie further back than the entry being written (n >= 1), so ascending order reads before it overwrites
  for (int s = 0; s < K - 1; ++s) {
    const int i = n - (K - 1) + s;
    S x;
    if (i >= 0) x = proj[(int64_t)(t0 + i) * ld + qkv_off + c];
    else x = start > 0 ? st[K - 1 + i] : from_f32<S>(0.f);
    st[s] = x;
  }
}

// A lane's value plus that of the lane a DPP pattern pairs it with (full-rate vector instructions, no LDS).
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// The sum over a row of 16 lanes, in every lane of it: neighbours, pairs of a quad, the quads of a half row
// (mirrored: all lanes of a quad hold the same sum by then), the two half rows.
__device__ __forceinline__ float row16_sum(float v) {
  v = dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  v = dpp_add<0x141>(v);   // row_half_mirror
  return dpp_add<0x140>(v);  // row_mirror
}
// The sum over 32 lanes (two DPP rows), in every lane of them.
__device__ __forceinline__ float half_wave_sum(float v) {
  v = row16_sum(v);
  return v + __shfl_xor(v, 16, WAVE);
}

// One request, one head and COLS columns of S a workgroup; the 32 lanes of half a wave share a column and own RPT
// consecutive rows each (D <= 32 RPT): a wave's work a token is what bounds a prompt of one request, so a column is
// spread over as many lanes as the sums' cost allows (16 lanes a column: 2,048 tokens of 16 heads of 128 x 128 in
// 550 us; 8 lanes and the sums taken one after the other: 1,066 us). With a = S^T k, b = S^T q and c = k . q taken from the state before the
// token, all three at once,   u = beta (v - g a),   o = g b + c u   (= (g S + k u^T)^T q),   S <- g S + k u^T:
// the rows are summed once a token instead of twice, and no product waits for the state's update.
template <int RPT>
__global__ void __launch_bounds__(256) delta_recurrence_kernel(
    const float* __restrict__ work, int64_t ldw, float* __restrict__ state, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_lens, float* __restrict__ out, int64_t ld_out,
    int G, int H, int D, int V) {
  constexpr int DP = 32 * RPT;
  __shared__ __attribute__((aligned(16))) float ks[CH][DP];
  __shared__ __attribute__((aligned(16))) float qs[CH][DP];
  __shared__ float vs[CH][COLS];
  __shared__ float bs[CH], gs[CH];
  // the request is the slowest index of the grid: the workgroups of one long request among many short ones then
  // spread over all XCDs (consecutive workgroups go to consecutive XCDs) instead of meeting on one
  const int b = blockIdx.z, h = blockIdx.y, cb = blockIdx.x;
  const int tid = threadIdx.x;
  const int rg = tid & 31, cj = tid >> 5;
  const int j = cb * COLS + cj;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  const int start = seq_lens[b] - n;
  const int g = h / (H / G);
  const int gd = 2 * G * D;
  const bool col_ok = j < V;
  float* sp = state + ((((int64_t)slots[b] * H + h) * V + (col_ok ? j : 0)) * D) + rg * RPT;
  float S[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) S[i] = (start > 0 && col_ok && rg * RPT + i < D) ? sp[i] : 0.f;

  // what a thread carries of the next chunk: RPT entries of k and of q, one of v, one of beta or g
  constexpr int PK = (CH * DP) / 256;
  float pk[PK], pq[PK], pv = 0.f, pbg = 0.f;
  const float* wk = work + (int64_t)t0 * ldw;
  auto fetch = [&](int ct) {
#pragma unroll
    for (int e = 0; e < PK; ++e) {
      const int idx = tid + e * 256;
      const int tok = idx / DP, d = idx % DP;
      const bool ok = ct + tok < n && d < D;
      const float* r = wk + (int64_t)(ct + tok) * ldw + g * D + d;
      pk[e] = ok ? r[G * D] : 0.f;
      pq[e] = ok ? r[0] : 0.f;
    }
    if (tid < CH * COLS) {
      const int tok = tid / COLS, c = tid % COLS;
      const int col = cb * COLS + c;
      pv = (ct + tok < n && col < V) ? wk[(int64_t)(ct + tok) * ldw + gd + h * V + col] : 0.f;
    }
    if (tid < 2 * CH) {
      const int tok = tid % CH;
      pbg = ct + tok < n ? wk[(int64_t)(ct + tok) * ldw + gd + H * V + (tid < CH ? 0 : H) + h] : 0.f;
    }
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
    if (tid < CH) bs[tid] = pbg;
    else if (tid < 2 * CH) gs[tid - CH] = pbg;
    __syncthreads();
    if (ct + CH < n) fetch(ct + CH);  // in flight while this chunk is worked through
    const int m = n - ct < CH ? n - ct : CH;
    // a token's operands are read from LDS while the token before is worked through
    float kr[RPT], qr[RPT], vt, bt_, gt;
    auto read = [&](int tok, float (&k_)[RPT], float (&q_)[RPT], float& v_, float& b_, float& g_) {
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        k_[i] = ks[tok][rg * RPT + i];
        q_[i] = qs[tok][rg * RPT + i];
      }
      v_ = vs[tok][cj];
      b_ = bs[tok];
      g_ = gs[tok];
    };
    read(0, kr, qr, vt, bt_, gt);
    for (int tok = 0; tok < m; ++tok) {
      float kn[RPT], qn[RPT], vn, bn, gn;
      read(tok + 1 < m ? tok + 1 : tok, kn, qn, vn, bn, gn);
      float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f, c0 = 0.f, c1 = 0.f;   // two chains a sum: a fixed order all the same
#pragma unroll
      for (int i = 0; i < RPT; i += 2) {
        a0 = __builtin_fmaf(S[i], kr[i], a0);
        b0 = __builtin_fmaf(S[i], qr[i], b0);
        c0 = __builtin_fmaf(kr[i], qr[i], c0);
        if (i + 1 < RPT) {
          a1 = __builtin_fmaf(S[i + 1], kr[i + 1], a1);
          b1 = __builtin_fmaf(S[i + 1], qr[i + 1], b1);
          c1 = __builtin_fmaf(kr[i + 1], qr[i + 1], c1);
        }
      }
      const float a = half_wave_sum(a0 + a1), bq = half_wave_sum(b0 + b1), c = half_wave_sum(c0 + c1);
      const float u = bt_ * (vt - gt * a);    // (g S)^T k = g (S^T k)
#pragma unroll
      for (int i = 0; i < RPT; ++i) S[i] = __builtin_fmaf(kr[i], u, gt * S[i]);
      if (rg == 0 && col_ok) out[(int64_t)(t0 + ct + tok) * ld_out + h * V + j] = __builtin_fmaf(c, u, gt * bq);
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        kr[i] = kn[i];
        qr[i] = qn[i];
      }
      vt = vn;
      bt_ = bn;
      gt = gn;
    }
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RPT; ++i)
      if (rg * RPT + i < D) sp[i] = S[i];
  }
}

template <class S>
__global__ void __launch_bounds__(WAVES * 64) delta_out_kernel(const float* __restrict__ o, int64_t ld_o,
                                                               const S* __restrict__ proj, int64_t ld, int64_t g_off,
                                                               const float* __restrict__ w, S* __restrict__ out,
                                                               int64_t ld_out, int64_t col_off, int H, int V, float eps,
                                                               float out_scale, int w_stride, int gate_kind) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * WAVES + wave;
  if (h >= H) return;
  constexpr int PER = MAX_HEAD / 64;
  float x[PER];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int d = lane + 64 * e;
    x[e] = d < V ? o[(int64_t)t * ld_o + h * V + d] : 0.f;
    ss = __builtin_fmaf(x[e], x[e], ss);
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)V + eps);
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int d = lane + 64 * e;
    if (d < V) {
      const float gl = to_f32(proj[(int64_t)t * ld + g_off + h * V + d]);
      const float gate = gate_kind == 1 ? sigmoid_f(gl) : silu_f(gl);
      out[(int64_t)t * ld_out + col_off + h * V + d] = from_f32<S>(x[e] * inv * w[h * w_stride + d] * gate * out_scale);
    }
  }
}


// ---- delta rule with a decay and a removal rate of its own for every key channel ------------------------------------
//
//   per token, per head:   S <- diag(w) S - (a * u) (u^T S) + k v^T   (both terms from the state before);   o = S^T r
//
// u = k / sqrt(sum k^2 + eps) the unit key, w in (0, 1) a decay and a in (0, 1) a removal rate a key channel. Column j
// of S goes its own way: s' = w * s - (a * u) A + k v_j with A = u . s, and o_j = r . s' = (r * w) . s - c1 A + c2 v_j
// with c1 = r . (a * u) and c2 = r . k, which depend on the token alone. So a token costs a column two sums (A and
// (r * w) . s), taken at once from the state before, and nothing waits for the update.
//
//   channel_delta_prep        one wave a (token, head): unit key, removal rate, decay
//                             w = exp(-rate * sigmoid(W2 tanh(l) + w0)) from the low-rank projection l, c1, c2. Float out.
//   channel_delta_recurrence  the layout of delta_recurrence: a request, a head and COLS columns a workgroup, 32 lanes a
//                             column, CH tokens' operands waiting in LDS while the next CH are on their way.
constexpr int MAX_LOW = 512;   // the largest inner size of the decay's low-rank projection

// work [T, ldw] float: rw (H D) | u (H D) | k (H D) | w (H D) | au (H D) | v (H D) | c1 (H) | c2 (H)
template <class S>
__global__ void __launch_bounds__(WAVES * 64) channel_delta_prep_kernel(
    const S* __restrict__ proj, int64_t ld, int64_t r_off, int64_t k_off, int64_t v_off, int64_t a_off, int64_t l_off,
    const float* __restrict__ a_bias, const float* __restrict__ w2, const float* __restrict__ w0, int low,
    float* __restrict__ work, int64_t ldw, int H, int D, float eps, float rate, const float* __restrict__ z_in,
    int64_t ld_z) {
  __shared__ float th[WAVES][MAX_LOW];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * WAVES + wave;
  if (h >= H) return;   // (no workgroup barrier below)
  const S* row = proj + (int64_t)t * ld;
  float* out = work + (int64_t)t * ldw;
  const int HD = H * D;
  if (!z_in) {
    for (int l = lane; l < low; l += 64) th[wave][l] = tanhf(to_f32(row[l_off + l]));
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  constexpr int PER = MAX_HEAD / 64;
  float kk[PER];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int d = lane + 64 * e;
    kk[e] = d < D ? to_f32(row[k_off + h * D + d]) : 0.f;
    ss = __builtin_fmaf(kk[e], kk[e], ss);
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) + eps);
  float c1 = 0.f, c2 = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int d = lane + 64 * e;
    if (d < D) {
      const int c = h * D + d;
      const float r = to_f32(row[r_off + c]);
      const float u = kk[e] * inv;
      const float a = sigmoid_f(to_f32(row[a_off + c]) + a_bias[c]);
      float z = w0[c];
      if (z_in) {   // the product with W2 was a matrix product of its own (steps of many rows)
        z += z_in[(int64_t)t * ld_z + c];
      } else {
        const float* w2r = w2 + (int64_t)c * low;
        for (int l = 0; l < low; ++l) z = __builtin_fmaf(w2r[l], th[wave][l], z);
      }
      const float w = expf(-rate * sigmoid_f(z));
      const float au = a * u;
      out[c] = r * w;
      out[HD + c] = u;
      out[2 * HD + c] = kk[e];
      out[3 * HD + c] = w;
      out[4 * HD + c] = au;
      out[5 * HD + c] = to_f32(row[v_off + c]);
      c1 = __builtin_fmaf(r, au, c1);
      c2 = __builtin_fmaf(r, kk[e], c2);
    }
  }
  c1 = wave_sum(c1);
  c2 = wave_sum(c2);
  if (lane == 0) {
    out[6 * HD + h] = c1;
    out[6 * HD + H + h] = c2;
  }
}

template <int RPT, int CHT>
__global__ void __launch_bounds__(256) channel_delta_recurrence_kernel(
    const float* __restrict__ work, int64_t ldw, float* __restrict__ state, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_lens, float* __restrict__ out, int64_t ld_out,
    int H, int D) {
  constexpr int DP = 32 * RPT;
  constexpr int NV = 5;   // rw, u, k, w, au
  __shared__ __attribute__((aligned(16))) float vec[NV][CHT][DP];
  __shared__ float vs[CHT][COLS];
  __shared__ float cs[2][CHT];
  const int b = blockIdx.z, h = blockIdx.y, cb = blockIdx.x;
  const int tid = threadIdx.x;
  const int rg = tid & 31, cj = tid >> 5;
  const int j = cb * COLS + cj;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  const int start = seq_lens[b] - n;
  const int HD = H * D;
  const bool col_ok = j < D;
  float* sp = state + ((((int64_t)slots[b] * H + h) * D + (col_ok ? j : 0)) * D) + rg * RPT;
  float S[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) S[i] = (start > 0 && col_ok && rg * RPT + i < D) ? sp[i] : 0.f;

  constexpr int PK = (CHT * DP) / 256;
  static_assert(PK >= 1 && (CHT * DP) % 256 == 0, "a chunk's vectors are dealt evenly among the threads");
  float pre[NV][PK], pv = 0.f, pc = 0.f;
  const float* wk = work + (int64_t)t0 * ldw;
  auto fetch = [&](int ct) {
#pragma unroll
    for (int e = 0; e < PK; ++e) {
      const int idx = tid + e * 256;
      const int tok = idx / DP, d = idx % DP;
      const bool ok = ct + tok < n && d < D;
      const float* r = wk + (int64_t)(ct + tok) * ldw + h * D + d;
#pragma unroll
      for (int v = 0; v < NV; ++v) pre[v][e] = ok ? r[v * HD] : 0.f;
    }
    if (tid < CHT * COLS) {
      const int tok = tid / COLS, c = tid % COLS;
      const int col = cb * COLS + c;
      pv = (ct + tok < n && col < D) ? wk[(int64_t)(ct + tok) * ldw + 5 * HD + h * D + col] : 0.f;
    }
    if (tid < 2 * CHT) {
      const int tok = tid % CHT;
      pc = ct + tok < n ? wk[(int64_t)(ct + tok) * ldw + 6 * HD + (tid < CHT ? 0 : H) + h] : 0.f;
    }
  };
  fetch(0);
  for (int ct = 0; ct < n; ct += CHT) {
    __syncthreads();  // the chunk before has been consumed
#pragma unroll
    for (int e = 0; e < PK; ++e) {
      const int idx = tid + e * 256;
#pragma unroll
      for (int v = 0; v < NV; ++v) vec[v][idx / DP][idx % DP] = pre[v][e];
    }
    if (tid < CHT * COLS) vs[tid / COLS][tid % COLS] = pv;
    if (tid < 2 * CHT) cs[tid / CHT][tid % CHT] = pc;
    __syncthreads();
    if (ct + CHT < n) fetch(ct + CHT);  // in flight while this chunk is worked through
    const int m = n - ct < CHT ? n - ct : CHT;
    for (int tok = 0; tok < m; ++tok) {
      float rw[RPT], u[RPT];
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        rw[i] = vec[0][tok][rg * RPT + i];
        u[i] = vec[1][tok][rg * RPT + i];
      }
      float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;   // two chains a sum: a fixed order all the same
#pragma unroll
      for (int i = 0; i < RPT; i += 2) {
        a0 = __builtin_fmaf(S[i], u[i], a0);
        b0 = __builtin_fmaf(S[i], rw[i], b0);
        if (i + 1 < RPT) {
          a1 = __builtin_fmaf(S[i + 1], u[i + 1], a1);
          b1 = __builtin_fmaf(S[i + 1], rw[i + 1], b1);
        }
      }
      const float vt = vs[tok][cj], c1 = cs[0][tok], c2 = cs[1][tok];
      const float A = half_wave_sum(a0 + a1), B = half_wave_sum(b0 + b1);
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        const float k = vec[2][tok][rg * RPT + i], w = vec[3][tok][rg * RPT + i], au = vec[4][tok][rg * RPT + i];
        S[i] = __builtin_fmaf(k, vt, __builtin_fmaf(-au, A, w * S[i]));
      }
      if (rg == 0 && col_ok) out[(int64_t)(t0 + ct + tok) * ld_out + h * D + j] = __builtin_fmaf(c2, vt, __builtin_fmaf(-c1, A, B));
    }
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RPT; ++i)
      if (rg * RPT + i < D) sp[i] = S[i];
  }
}

}  // namespace

// proj [T, ld]: the step's fused projection; q (G D) | k (G D) | v (H V) lie together from column qkv_off, the H
// step-size logits at b_off, the H decay logits at a_off. taps [2 G D + H V, K] float, the last column the current
// token's. a_log, dt_bias [H] float. conv_state [slots, 2 G D + H V, K - 1] in the step's dtype (unused with K = 1).
// work [T, ldw] float, ldw >= 2 G D + H V + 2 H.
extern "C" int dinfer_delta_prep(int dtype, const void* proj, int64_t ld, int64_t qkv_off, int64_t b_off, int64_t a_off,
                                 const float* taps, const float* taps_t, const float* a_log, const float* dt_bias,
                                 const void* conv_state, const int32_t* state_slots, const int32_t* cu_seqlens,
                                 const int32_t* seq_lens, float* work, int64_t ldw, int num_reqs, int64_t tokens, int G,
                                 int H, int D, int V, int K, float eps, float q_scale, hipStream_t stream) {
  // taps_t (may be null): the taps once more as [K, channels], for the kernel that takes 8 channels a lane
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (G <= 0 || H <= 0 || H % G || D <= 0 || V <= 0 || K <= 0 || tokens > 0x7fffffff ||
      ldw < 2 * (int64_t)G * D + (int64_t)H * V + 2 * H)
    return ERR_BAD_SHAPE;
  if (D > MAX_HEAD || V > MAX_HEAD || K > MAX_TAPS) return ERR_UNSUPPORTED;
  const bool lanes_even = D >= 32 && D <= 512 && (D & (D - 1)) == 0 && V % 8 == 0;
  if (taps_t && lanes_even && ld % 8 == 0 && qkv_off % 8 == 0 && ldw % 4 == 0 && ((uintptr_t)proj % 16) == 0 &&
      ((uintptr_t)work % 16) == 0 && ((uintptr_t)taps_t % 16) == 0) {
    const int pieces = (2 * G * D + H * V) / 8 + H;
    const dim3 grid((unsigned)tokens, (unsigned)((pieces + 255) / 256));
    DINFER_DISPATCH_DTYPE(dtype, {
      delta_prep_vec_kernel<S><<<grid, 256, 0, stream>>>((const S*)proj, ld, qkv_off, b_off, a_off, taps_t, a_log, dt_bias,
                                                         (const S*)conv_state, state_slots, cu_seqlens, seq_lens, work,
                                                         ldw, num_reqs, G, H, D, V, K, eps, q_scale);
    });
    return launch_status();
  }
  const dim3 grid((unsigned)tokens, (unsigned)((2 * G + H + 1 + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    delta_prep_kernel<S><<<grid, WAVES * 64, 0, stream>>>((const S*)proj, ld, qkv_off, b_off, a_off, taps, a_log,
                                                          dt_bias, (const S*)conv_state, state_slots, cu_seqlens,
                                                          seq_lens, work, ldw, num_reqs, G, H, D, V, K, eps, q_scale);
  });
  return launch_status();
}

extern "C" int dinfer_delta_conv_update(int dtype, const void* proj, int64_t ld, int64_t qkv_off, void* conv_state,
                                        const int32_t* state_slots, const int32_t* cu_seqlens, const int32_t* seq_lens,
                                        int num_reqs, int channels, int K, hipStream_t stream) {
  if (num_reqs <= 0 || K <= 1) return OK;
  if (channels <= 0 || K > MAX_TAPS) return ERR_BAD_SHAPE;
  const dim3 grid((unsigned)num_reqs, (unsigned)((channels + 255) / 256));
  DINFER_DISPATCH_DTYPE(dtype, {
    delta_conv_update_kernel<S><<<grid, 256, 0, stream>>>((const S*)proj, ld, qkv_off, (S*)conv_state, state_slots,
                                                          cu_seqlens, seq_lens, channels, K);
  });
  return launch_status();
}

// state [slots, H, V, D] float (S transposed); out [T, ld_out] float, head h at column h V.
extern "C" int dinfer_delta_recurrence(const float* work, int64_t ldw, float* state, const int32_t* state_slots,
                                       const int32_t* cu_seqlens, const int32_t* seq_lens, float* out, int64_t ld_out,
                                       int num_reqs, int G, int H, int D, int V, hipStream_t stream) {
  if (num_reqs <= 0) return OK;
  if (G <= 0 || H <= 0 || H % G || D <= 0 || V <= 0 || num_reqs > 65535 || H > 65535) return ERR_BAD_SHAPE;
  if (D > 256) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)((V + COLS - 1) / COLS), (unsigned)H, (unsigned)num_reqs);
#define DELTA_REC(R_)                                                                                               \
  delta_recurrence_kernel<R_><<<grid, 256, 0, stream>>>(work, ldw, state, state_slots, cu_seqlens, seq_lens, out, \
                                                        ld_out, G, H, D, V)
  if (D <= 32) DELTA_REC(1);
  else if (D <= 64) DELTA_REC(2);
  else if (D <= 128) DELTA_REC(4);
  else DELTA_REC(8);
#undef DELTA_REC
  return launch_status();
}

// out[t, col_off + h V + d] = o[t, h V + d] / sqrt(mean_d o^2 + eps) * w[d] * silu(proj[t, g_off + h V + d]) * out_scale
// w_per_head: w holds H V gains, a head's own at h V; gate_kind: 0 silu, 1 the logistic function.
extern "C" int dinfer_delta_out(int dtype, const float* o, int64_t ld_o, const void* proj, int64_t ld, int64_t g_off,
                                const float* w, void* out, int64_t ld_out, int64_t col_off, int64_t tokens, int H, int V,
                                float eps, float out_scale, int w_per_head, int gate_kind, hipStream_t stream) {
  if (gate_kind != 0 && gate_kind != 1) return ERR_UNSUPPORTED;
  if (tokens <= 0) return OK;
  if (H <= 0 || V <= 0 || tokens > 0x7fffffff) return ERR_BAD_SHAPE;
  if (V > MAX_HEAD) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((H + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    delta_out_kernel<S><<<grid, WAVES * 64, 0, stream>>>(o, ld_o, (const S*)proj, ld, g_off, w, (S*)out, ld_out,
                                                         col_off, H, V, eps, out_scale, w_per_head ? V : 0, gate_kind);
  });
  return launch_status();
}

// The rule with a decay and a removal rate a key channel (see above). proj [T, ld]: r, k, v (H D each) at their columns,
// the H D removal logits at a_off, the `low` entries of the decay's inner projection at l_off. a_bias, w0 [H D] float,
// w2 [H D, low] float. work [T, ldw] float, ldw >= 6 H D + 2 H. z (may be null) [T, ld_z] float: W2 tanh(.) as a
// matrix product of the caller's made it; then the kernel only adds w0.
extern "C" int dinfer_channel_delta_prep(int dtype, const void* proj, int64_t ld, int64_t r_off, int64_t k_off,
                                         int64_t v_off, int64_t a_off, int64_t l_off, const float* a_bias,
                                         const float* w2, const float* w0, int low, float* work, int64_t ldw,
                                         int64_t tokens, int H, int D, float eps, float rate, const float* z,
                                         int64_t ld_z, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (H <= 0 || D <= 0 || low <= 0 || tokens > 0x7fffffff || ldw < 6LL * H * D + 2 * H) return ERR_BAD_SHAPE;
  if (D > MAX_HEAD || low > MAX_LOW) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((H + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    channel_delta_prep_kernel<S><<<grid, WAVES * 64, 0, stream>>>((const S*)proj, ld, r_off, k_off, v_off, a_off, l_off,
                                                                  a_bias, w2, w0, low, work, ldw, H, D, eps, rate, z,
                                                                  ld_z);
  });
  return launch_status();
}

// state [slots, H, D, D] float (a head's matrix transposed: [value, key]); out [T, ld_out] float, head h at h D.
extern "C" int dinfer_channel_delta_recurrence(const float* work, int64_t ldw, float* state, const int32_t* state_slots,
                                               const int32_t* cu_seqlens, const int32_t* seq_lens, float* out,
                                               int64_t ld_out, int num_reqs, int H, int D, hipStream_t stream) {
  if (num_reqs <= 0) return OK;
  if (H <= 0 || D <= 0 || num_reqs > 65535 || H > 65535) return ERR_BAD_SHAPE;
  if (D > 256) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)((D + COLS - 1) / COLS), (unsigned)H, (unsigned)num_reqs);
#define CHANNEL_REC(R_, C_)                                                                                          \
  channel_delta_recurrence_kernel<R_, C_><<<grid, 256, 0, stream>>>(work, ldw, state, state_slots, cu_seqlens,       \
                                                                    seq_lens, out, ld_out, H, D)
  if (D <= 32) CHANNEL_REC(1, 16);
  else if (D <= 64) CHANNEL_REC(2, 16);
  else if (D <= 128) CHANNEL_REC(4, 16);
  else CHANNEL_REC(8, 8);
#undef CHANNEL_REC
  return launch_status();
}
