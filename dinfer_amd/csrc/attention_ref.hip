// Plain paged attention for any head size, group size, page size and storage
// type: the kernel of the 32-bit path and the reference beside the MFMA
// kernels. One wave per (token, query head); keys are visited in ascending
// order in tiles of 64, so a row's arithmetic depends only on its own position
// and never on how the step was cut or batched.
//
//   row i of request b has position p = seq_len[b] - q_len[b] + i and sees the
//   keys j in [max(0, p - window + 1), p]  (window 0: all keys up to p);
//   s_j = scale * <q, k_j>;  P = softmax(s);  o = sum_j P_j v_j   (all float)
//
// Options (dinfer_attn_paged_ext; each is off at its zero):
//   keep_first F   the keys j < F stay visible after the window has passed them (they keep their positions);
//   sinks          one float a query head: exp(sink_h) is added to the softmax's denominator once; it has no key, no
//                  value and is not scaled;
//   slope_exp E    s_j -= 2^(-E (h + 1) / H) * (p - j): a bias that grows with the distance, steeper for low heads;
//   v_dim          the value size where it differs from the key size;
//   values in the key pages (v_cache null): a layer whose values are its keys stores them once;
//   out_scale      o is multiplied by it on store.
//
// K and V are read from the cache pages through the request's block table
// (K page [Hkv][ceil(D / 8)][page][8], V page [Hkv][D][page]); the step's own tokens were
// written there before this kernel runs.
//
// Reference behaviour: crates/kernels/cuda/gqa.cu:1037-1118 (plain paged
// kernel: causal inclusive, query head h reads kv head h / G, online softmax,
// 0 when nothing was summed).
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int MAX_D = 512;
constexpr int WAVES = 4;

template <class S>
__global__ void __launch_bounds__(WAVES * 64) attn_paged_ref_kernel(
    const S* __restrict__ q, int64_t ld_q, S* __restrict__ out, int64_t ld_out, const S* __restrict__ k_cache,
    const S* __restrict__ v_cache, const int32_t* __restrict__ block_table, int64_t max_blocks,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_lens, int num_reqs, float scale,
    int window, int H, int Hkv, int D, int page, int keep_first, const float* __restrict__ sinks, float slope_exp,
    int Dv, float out_scale) {
  __shared__ float qs[WAVES][MAX_D];
  __shared__ float ps[WAVES][64];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * WAVES + wave;
  const bool live = h < H;

  // the request of token t: cu[b] <= t < cu[b+1]
  int lo_b = 0, hi_b = num_reqs - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (cu_seqlens[mid] <= t) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int q_len = cu_seqlens[b + 1] - cu_seqlens[b];
  const int p = seq_lens[b] - q_len + (t - cu_seqlens[b]);
  const int first_key = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int32_t* bt = block_table + (int64_t)b * max_blocks;
  const int hk = live ? h / (H / Hkv) : 0;
  const int Dp = (D + 7) & ~7;  // a head's keys fill whole 8-entry pieces of a page (the last one padded)
  const float slope = slope_exp != 0.f ? exp2f(-slope_exp * (float)(h + 1) / (float)H) : 0.f;
  // two runs of keys: the kept first ones that the window has passed, then the window itself
  const int kept = keep_first < first_key ? keep_first : first_key;

  if (live) {
    const S* qr = q + (int64_t)t * ld_q + (int64_t)h * D;
    for (int d = lane; d < D; d += 64) qs[wave][d] = to_f32(qr[d]);
  }
  __syncthreads();

  constexpr int NC = MAX_D / 64;
  float o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) o[c] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int run = kept > 0 ? 0 : 1; run < 2; ++run)
  for (int j0 = run ? first_key : 0, last = run ? p : kept - 1; j0 <= last; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (live && j <= last) {
      const int blk = bt[j / page];
      const S* kr = k_cache + ((int64_t)blk * Hkv + hk) * page * Dp;  // the head's page
      const int off = j % page;
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc += qs[wave][d] * to_f32(kr[k_page_offset(off, d, page)]);
      s = acc * scale - slope * (float)(p - j);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = (live && j <= last) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // m = -inf on the first tile: alpha = 0
    l = l * alpha + wave_sum(pj);
    m = m_new;
    __syncthreads();  // the previous tile's ps[] has been consumed
    ps[wave][lane] = pj;
    __syncthreads();
    if (live) {
      const int n = last - j0 + 1 < 64 ? last - j0 + 1 : 64;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = lane + 64 * c;
        if (d < Dv) {
          float acc = o[c] * alpha;
          for (int jj = 0; jj < n; ++jj) {
            const int key = j0 + jj;
            const int blk = bt[key / page];
            const S* vr = v_cache ? v_cache + (((int64_t)blk * Hkv + hk) * Dv + d) * page + (key % page)
                                  : k_cache + ((int64_t)blk * Hkv + hk) * page * Dp + k_page_offset(key % page, d, page);
            acc += ps[wave][jj] * to_f32(*vr);
          }
          o[c] = acc;
        }
      }
    }
  }
  if (live && sinks) {  // the sink joins the denominator as one more term
    const float sk = sinks[h];
    const float m_new = fmaxf(m, sk);
    const float alpha = expf(m - m_new);
    l = l * alpha + expf(sk - m_new);
#pragma unroll
    for (int c = 0; c < NC; ++c) o[c] *= alpha;
  }
  if (live) {
    S* orow = out + (int64_t)t * ld_out + (int64_t)h * Dv;
    const float inv = l > 0.f ? out_scale / l : 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < Dv) orow[d] = from_f32<S>(o[c] * inv);
    }
  }
}

// Differential attention: a query head holds two queries of D entries, [first map | second map], and so does a key
// head; each map is a softmax attention of its own over the same values, and the head's output is
//   o = a1 - lambda a2,   o <- o / sqrt(mean(o^2) + eps) * post      (the mean over the head's Dv values)
// One wave per (token, query head) walks the keys once and keeps both maps' (max, sum, output). The key pages hold
// heads of 2 D entries, the value pages heads of Dv.
template <class S>
__global__ void __launch_bounds__(WAVES * 64) attn_paged_diff_kernel(
    const S* __restrict__ q, int64_t ld_q, S* __restrict__ out, int64_t ld_out, const S* __restrict__ k_cache,
    const S* __restrict__ v_cache, const int32_t* __restrict__ block_table, int64_t max_blocks,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_lens, int num_reqs, float scale,
    int window, int H, int Hkv, int D, int page, int Dv, float lambda, float eps, float post) {
  __shared__ float qs[WAVES][MAX_D];
  __shared__ float ps[WAVES][2][64];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * WAVES + wave;
  const bool live = h < H;

  int lo_b = 0, hi_b = num_reqs - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (cu_seqlens[mid] <= t) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int q_len = cu_seqlens[b + 1] - cu_seqlens[b];
  const int p = seq_lens[b] - q_len + (t - cu_seqlens[b]);
  const int first_key = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int32_t* bt = block_table + (int64_t)b * max_blocks;
  const int hk = live ? h / (H / Hkv) : 0;
  const int D2 = 2 * D;
  const int Dp = (D2 + 7) & ~7;

  if (live) {
    const S* qr = q + (int64_t)t * ld_q + (int64_t)h * D2;
    for (int d = lane; d < D2; d += 64) qs[wave][d] = to_f32(qr[d]);
  }
  __syncthreads();

  constexpr int NC = MAX_D / 64;
  float o1[NC], o2[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) o1[c] = o2[c] = 0.f;
  float m1 = -INFINITY, l1 = 0.f, m2 = -INFINITY, l2 = 0.f;

  for (int j0 = first_key; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s1 = -INFINITY, s2 = -INFINITY;
    if (live && j <= p) {
      const int blk = bt[j / page];
      const S* kr = k_cache + ((int64_t)blk * Hkv + hk) * page * Dp;
      const int off = j % page;
      float acc1 = 0.f, acc2 = 0.f;
      for (int d = 0; d < D; ++d) {
        acc1 += qs[wave][d] * to_f32(kr[k_page_offset(off, d, page)]);
        acc2 += qs[wave][D + d] * to_f32(kr[k_page_offset(off, D + d, page)]);
      }
      s1 = acc1 * scale;
      s2 = acc2 * scale;
    }
    const float n1 = fmaxf(m1, wave_max(s1)), n2 = fmaxf(m2, wave_max(s2));
    const float p1 = (live && j <= p) ? expf(s1 - n1) : 0.f, p2 = (live && j <= p) ? expf(s2 - n2) : 0.f;
    const float al1 = expf(m1 - n1), al2 = expf(m2 - n2);
    l1 = l1 * al1 + wave_sum(p1);
    l2 = l2 * al2 + wave_sum(p2);
    m1 = n1;
    m2 = n2;
    __syncthreads();
    ps[wave][0][lane] = p1;
    ps[wave][1][lane] = p2;
    __syncthreads();
    if (live) {
      const int n = p - j0 + 1 < 64 ? p - j0 + 1 : 64;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = lane + 64 * c;
        if (d < Dv) {
          float x1 = o1[c] * al1, x2 = o2[c] * al2;
          for (int jj = 0; jj < n; ++jj) {
            const int key = j0 + jj;
            const int blk = bt[key / page];
            const float v = to_f32(v_cache[(((int64_t)blk * Hkv + hk) * Dv + d) * page + (key % page)]);
            x1 += ps[wave][0][jj] * v;
            x2 += ps[wave][1][jj] * v;
          }
          o1[c] = x1;
          o2[c] = x2;
        }
      }
    }
  }
  if (live) {
    const float i1 = l1 > 0.f ? 1.f / l1 : 0.f, i2 = l2 > 0.f ? lambda / l2 : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      o1[c] = d < Dv ? o1[c] * i1 - o2[c] * i2 : 0.f;
      ss += o1[c] * o1[c];
    }
    const float inv = post / sqrtf(wave_sum(ss) / (float)Dv + eps);
    S* orow = out + (int64_t)t * ld_out + (int64_t)h * Dv;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < Dv) orow[d] = from_f32<S>(o1[c] * inv);
    }
  }
}

// The end of a differential head where its two maps were computed as heads of their own (side by side, the first map's
// Dv values and then the second's): o = a1 - lambda a2, o <- o / sqrt(mean(o^2) + eps) * post. One wave per (token, head).
template <class S>
__global__ void __launch_bounds__(WAVES * 64) diff_combine_kernel(const S* __restrict__ in, int64_t ld_in, S* __restrict__ out,
                                                                  int64_t ld_out, int H, int Dv, float lambda, float eps,
                                                                  float post) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * WAVES + wave;
  if (h >= H) return;
  const S* a = in + (int64_t)t * ld_in + (int64_t)2 * h * Dv;
  constexpr int NC = MAX_D / 64;
  float o[NC];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int d = lane + 64 * c;
    o[c] = d < Dv ? to_f32(a[d]) - lambda * to_f32(a[Dv + d]) : 0.f;
    ss += o[c] * o[c];
  }
  const float inv = post / sqrtf(wave_sum(ss) / (float)Dv + eps);
  S* orow = out + (int64_t)t * ld_out + (int64_t)h * Dv;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int d = lane + 64 * c;
    if (d < Dv) orow[d] = from_f32<S>(o[c] * inv);
  }
}

}  // namespace

// q [T, ld_q] (head h at column h*D), out [T, ld_out]; block_table [num_reqs, max_blocks];
// cu_seqlens [num_reqs+1] prefix sums of the rows per request; seq_lens [num_reqs]
// lengths after this step.
extern "C" int dinfer_attn_paged_ref(int dtype, const void* q, int64_t ld_q, void* out, int64_t ld_out,
                                     const void* k_cache, const void* v_cache, const int32_t* block_table,
                                     int64_t max_blocks, const int32_t* cu_seqlens, const int32_t* seq_lens,
                                     int num_reqs, int64_t tokens, float scale, int window, int heads, int kv_heads,
                                     int head_dim, int page_size, hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0 || page_size <= 0 || max_blocks <= 0 ||
      window < 0 || tokens > 0x7fffffff)
    return ERR_BAD_SHAPE;
  if (head_dim > MAX_D) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((heads + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    attn_paged_ref_kernel<S><<<grid, WAVES * 64, 0, stream>>>(
        (const S*)q, ld_q, (S*)out, ld_out, (const S*)k_cache, (const S*)v_cache, block_table, max_blocks, cu_seqlens,
        seq_lens, num_reqs, scale, window, heads, kv_heads, head_dim, page_size, 0, nullptr, 0.f, head_dim, 1.f);
  });
  return launch_status();
}

// The same with the options of the header. out [T, ld_out] holds head h at column h * v_dim. v_cache null: the values
// are the keys and are read from the key pages (v_dim must equal head_dim).
extern "C" int dinfer_attn_paged_ext(int dtype, const void* q, int64_t ld_q, void* out, int64_t ld_out,
                                     const void* k_cache, const void* v_cache, const int32_t* block_table,
                                     int64_t max_blocks, const int32_t* cu_seqlens, const int32_t* seq_lens,
                                     int num_reqs, int64_t tokens, float scale, int window, int keep_first,
                                     const float* sinks, float slope_exp, int heads, int kv_heads, int head_dim,
                                     int v_dim, int page_size, float out_scale, hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0 || v_dim <= 0 || page_size <= 0 ||
      max_blocks <= 0 || window < 0 || keep_first < 0 || tokens > 0x7fffffff || (!v_cache && v_dim != head_dim))
    return ERR_BAD_SHAPE;
  if (head_dim > MAX_D || v_dim > MAX_D) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((heads + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    attn_paged_ref_kernel<S><<<grid, WAVES * 64, 0, stream>>>(
        (const S*)q, ld_q, (S*)out, ld_out, (const S*)k_cache, (const S*)v_cache, block_table, max_blocks, cu_seqlens,
        seq_lens, num_reqs, scale, window, heads, kv_heads, head_dim, page_size, window > 0 ? keep_first : 0, sinks,
        slope_exp, v_dim, out_scale);
  });
  return launch_status();
}

// Differential attention (see the kernel). q [T, ld_q]: head h at column 2 h head_dim, first map then second; the key
// pages hold kv_heads heads of 2 head_dim entries, the value pages heads of v_dim; out [T, ld_out], head h at h v_dim.
extern "C" int dinfer_attn_paged_diff(int dtype, const void* q, int64_t ld_q, void* out, int64_t ld_out,
                                      const void* k_cache, const void* v_cache, const int32_t* block_table,
                                      int64_t max_blocks, const int32_t* cu_seqlens, const int32_t* seq_lens,
                                      int num_reqs, int64_t tokens, float scale, int window, int heads, int kv_heads,
                                      int head_dim, int v_dim, int page_size, float lambda, float eps, float post,
                                      hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0 || v_dim <= 0 || page_size <= 0 ||
      max_blocks <= 0 || window < 0 || tokens > 0x7fffffff || !v_cache)
    return ERR_BAD_SHAPE;
  if (2 * head_dim > MAX_D || v_dim > MAX_D) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((heads + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    attn_paged_diff_kernel<S><<<grid, WAVES * 64, 0, stream>>>(
        (const S*)q, ld_q, (S*)out, ld_out, (const S*)k_cache, (const S*)v_cache, block_table, max_blocks, cu_seqlens,
        seq_lens, num_reqs, scale, window, heads, kv_heads, head_dim, page_size, v_dim, lambda, eps, post);
  });
  return launch_status();
}

// in [T, ld_in]: head h's two maps at columns 2 h v_dim and (2 h + 1) v_dim; out [T, ld_out]: head h at h v_dim.
extern "C" int dinfer_diff_combine(int dtype, const void* in, int64_t ld_in, void* out, int64_t ld_out, int64_t tokens,
                                   int heads, int v_dim, float lambda, float eps, float post, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (heads <= 0 || v_dim <= 0 || tokens > 0x7fffffff || ld_in < 2LL * heads * v_dim || ld_out < (int64_t)heads * v_dim)
    return ERR_BAD_SHAPE;
  if (v_dim > MAX_D) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((heads + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    diff_combine_kernel<S><<<grid, WAVES * 64, 0, stream>>>((const S*)in, ld_in, (S*)out, ld_out, heads, v_dim, lambda, eps,
                                                            post);
  });
  return launch_status();
}
