// Latent attention: every token keeps one vector of R + dr numbers that all heads share (the RMS-normed latent c
// [R] and one rotated key part kr [dr]); a head's unrotated key is Wuk_h c and its value Wuv_h c. The products
// with Wuk and Wuv are moved to the query side (the "absorbed" form), so the kernels here never expand a key:
//
//   qa_h = [ Wuk_h^T qn_h | rot(qr_h) ]          (R + dr numbers a head, made before these kernels run)
//   s_j  = scale * < qa_h , [c_j | kr_j] >       j <= p  (and j > p - window, where a window is given)
//   ol_h = sum_j softmax(s)_j c_j                (R numbers a head; the caller multiplies by Wuv_h)
//
// which is attention with one shared key/value head whose keys are R + dr wide and whose values are the first R
// numbers of the same row. Cache pages: [blocks][page][R + dr], one row a token; for the matrix cores a second copy of
// the latents, transposed a page at a time, [blocks][R][page]: the product with the values contracts over the keys, and
// an MFMA operand wants consecutive entries of the contraction in one lane, so consecutive keys of one latent entry
// must lie next to each other (the same reason the key/value cache keeps its values transposed).
//
//   latent_post    from the step's projections: RMS norm of the latent (float), rotation of the shared key part and
//                  of every head's rotated query part (pairs (2i, 2i+1), float angles from a table), the latent row
//                  written to its cache slot, the rotated query part written beside the absorbed part
//   latent_attn_ref  one wave per (token, head), keys in ascending tiles of 64, float arithmetic, any sizes: the
//                  kernel of the 32-bit path and the reference beside the MFMA kernel
//   latent_attn_mfma bf16: a workgroup takes 16 (token, head) rows of one request (heads fastest); its four waves
//                  deal the blocks of 32 keys among themselves in contiguous runs, each keeps its own (max, sum,
//                  output), and they meet in LDS at the end. Scores are computed transposed (keys x rows), so that a
//                  lane's eight weights are exactly its operand of the product with the values: nothing crosses lanes
//                  between the two products, and a lane keeps the softmax state of one row. With `splits` > 1 the
//                  keys of a request are cut into that many parts on the device (steps of single rows) and a merge
//                  kernel joins them; the launch shape follows the step's counts alone.
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int MAX_DK = 1280;  // R + dr
constexpr int MAX_R = 1024;
constexpr int WAVES = 4;

// ---- projections -> absorbed-query buffer and cache -------------------------------------------------------------
template <class S>
__global__ void __launch_bounds__(256) latent_post_kernel(
    const S* __restrict__ proj, int64_t ld, int q_off, int c_off, int H, int dn, int dr, int R,
    const void* __restrict__ gain, int wf32, float eps, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_sin, int rot, S* __restrict__ qa, int64_t ld_qa, S* __restrict__ cache,
    S* __restrict__ cache_t, int page, const int64_t* __restrict__ slots, int style, const S* __restrict__ qsrc,
    int64_t ld_qs) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const S* row = proj + t * ld;
  const S* qrow = qsrc ? qsrc + t * ld_qs : row;   // the queries may come from a product of their own
  const int pos = positions[t];
  const float* cs = cos_sin ? cos_sin + (int64_t)pos * rot : nullptr;
  const int half = rot / 2;
  // every head's rotated query part
  const int pairs = dr / 2;
  for (int i = threadIdx.x; i < H * pairs; i += blockDim.x) {
    const int h = i / pairs, j = i - h * pairs;
    // style 1: entries (2j, 2j+1) pair up; style 0: entry j pairs with j + rot/2 (the entries from rot on, which do
    // not turn, are walked two by two in either style)
    const bool halves = style == 0 && j < half;
    const int ia = halves ? j : 2 * j, ib = halves ? j + half : 2 * j + 1;
    const S* src = qrow + q_off + (int64_t)h * (dn + dr) + dn;
    float u = to_f32(src[ia]), v = to_f32(src[ib]);
    if (cs && j < half) {
      const float c = cs[j], s = cs[half + j];
      const float a = rotated_first(u, v, c, s), b = rotated_second(u, v, c, s);
      u = a; v = b;
    }
    S* dst = qa + t * ld_qa + (int64_t)h * (R + dr) + R;
    dst[ia] = from_f32<S>(u);
    dst[ib] = from_f32<S>(v);
  }
  if (dr & 1) {   // an odd last entry passes unchanged
    for (int h = threadIdx.x; h < H; h += blockDim.x)
      qa[t * ld_qa + (int64_t)h * (R + dr) + R + dr - 1] = qrow[q_off + (int64_t)h * (dn + dr) + dn + dr - 1];
  }
  if (c_off < 0 || !slots) return;
  const int64_t slot = slots[t];
  if (slot < 0) return;   // (uniform over the workgroup)
  const S* c = row + c_off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) ss = add_square(ss, to_f32(c[i]));
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)R + eps);
  S* dst = cache + slot * (int64_t)(R + dr);
  S* dst_t = cache_t ? cache_t + (slot / page) * (int64_t)R * page + (slot % page) : nullptr;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const S v = from_f32<S>(to_f32(c[i]) * inv * ld_param<S>(gain, i, wf32));
    dst[i] = v;
    if (dst_t) dst_t[(int64_t)i * page] = v;
  }
  for (int j = threadIdx.x; j < pairs; j += blockDim.x) {
    const bool halves = style == 0 && j < half;
    const int ia = halves ? j : 2 * j, ib = halves ? j + half : 2 * j + 1;
    float u = to_f32(c[R + ia]), v = to_f32(c[R + ib]);
    if (cs && j < half) {
      const float co = cs[j], si = cs[half + j];
      const float a = rotated_first(u, v, co, si), b = rotated_second(u, v, co, si);
      u = a; v = b;
    }
    dst[R + ia] = from_f32<S>(u);
    dst[R + ib] = from_f32<S>(v);
  }
  if ((dr & 1) && threadIdx.x == 0) dst[R + dr - 1] = c[R + dr - 1];
}

// ---- plain attention over the latent pages ----------------------------------------------------------------------
template <class S>
__global__ void __launch_bounds__(WAVES * 64) latent_attn_ref_kernel(
    const S* __restrict__ qa, int64_t ld_qa, S* __restrict__ out, int64_t ld_out, const S* __restrict__ cache,
    const int32_t* __restrict__ block_table, int64_t max_blocks, const int32_t* __restrict__ cu_seqlens,
    const int32_t* __restrict__ seq_lens, int num_reqs, float scale, int window, int H, int R, int dr, int page) {
  extern __shared__ float lds[];
  const int DK = R + dr;
  float* qs = lds;                   // [WAVES][DK]
  float* ps = lds + WAVES * DK;      // [WAVES][64]
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
  if (live) {
    const S* qr = qa + (int64_t)t * ld_qa + (int64_t)h * DK;
    for (int d = lane; d < DK; d += 64) qs[wave * DK + d] = to_f32(qr[d]);
  }
  __syncthreads();
  constexpr int NC = MAX_R / 64;
  float o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) o[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int j0 = first_key; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (live && j <= p) {
      const S* kr = cache + ((int64_t)bt[j / page] * page + (j % page)) * DK;
      float acc = 0.f;
      for (int d = 0; d < DK; ++d) acc = fmaf(qs[wave * DK + d], to_f32(kr[d]), acc);
      s = acc * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = (live && j <= p) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(pj);
    m = m_new;
    __syncthreads();
    ps[wave * 64 + lane] = pj;
    __syncthreads();
    if (live) {
      const int n = p - j0 + 1 < 64 ? p - j0 + 1 : 64;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = lane + 64 * c;
        if (d < R) {
          float acc = o[c] * alpha;
          for (int jj = 0; jj < n; ++jj) {
            const int key = j0 + jj;
            acc = fmaf(ps[wave * 64 + jj], to_f32(cache[((int64_t)bt[key / page] * page + (key % page)) * DK + d]), acc);
          }
          o[c] = acc;
        }
      }
    }
  }
  if (live) {
    S* orow = out + (int64_t)t * ld_out + (int64_t)h * R;
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < R) orow[d] = from_f32<S>(o[c] * inv);
    }
  }
}


// ---- attention over the latent pages on the matrix cores --------------------------------------------------------
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float exp2_of(float x) { return __builtin_amdgcn_exp2f(x); }

// NT: tiles of 16 latent entries (R <= 16 NT, R a multiple of 16); the key rows are cut into NT / 2 + 4 chunks of 32
// entries (dr <= 128). v_mfma_f32_16x16x32_bf16: lane l holds row (first operand) or column (second) l % 16 and the 8
// entries of the contraction that belong to group l / 16; of the result, column l % 16 and rows 4 (l / 16) .. + 3.
//   scores   first operand 16 keys x 32 key entries (rows of the cache, 16 bytes a lane), second the queries;
//            lane l gets, for query row l % 16, rows 4 (l / 16) .. + 3 of each of the block's two key tiles
//   values   contraction over the block's 32 keys in the order in which a lane holds its weights, which the rows of the
//            two key tiles are numbered for (see the loop): group g holds keys 8g .. 8g+7; first operand 16 latent
//            entries x those keys (16 bytes of a transposed page), second the weights; the result is O^T: lane l holds
//            query row l % 16 and latent entries 16 tile + 4 (l / 16) .. + 3.
// SOLO: steps with prompt portions: every wave takes a row tile of its own and walks all its keys (the four waves of
// a workgroup take consecutive tiles, so they ask for the same keys at about the same time and meet in the cache);
// otherwise (steps of single rows) the four waves share one row tile and deal its keys among themselves.
template <int NT, bool SOLO>
__global__ void __launch_bounds__(256) latent_attn_mfma_kernel(
    const bf16* __restrict__ qa, int64_t ld_qa, bf16* __restrict__ out, int64_t ld_out, float* __restrict__ part,
    const bf16* __restrict__ cache, const bf16* __restrict__ cache_t, const int32_t* __restrict__ block_table,
    int64_t max_blocks, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_lens, int num_reqs,
    float scale_log2, int window, int H, int R, int dr, int page, int splits) {
  constexpr int NC = NT / 2 + 4;
  constexpr int KG = 4, VG = NT < 8 ? NT : 8;   // loads of keys (x 2 tiles) and of values in flight before a product waits (more cost registers and with them the second wave of a SIMD: measured slower)
  extern __shared__ float meet[];   // [16][R + 4]: one wave's output, max and sum on their way to wave 0
  // which request and which of its row tiles: 64 requests at a time, one a lane, counted with a prefix sum over the wave
  int tile = SOLO ? blockIdx.x * 4 + (int)(threadIdx.x >> 6) : blockIdx.x, b = -1, q_len = 0;
  {
    const int ln = threadIdx.x & 63;
    for (int b0 = 0; b0 < num_reqs && b < 0; b0 += 64) {
      const int mine = b0 + ln < num_reqs ? cu_seqlens[b0 + ln + 1] - cu_seqlens[b0 + ln] : 0;
      int upto = (mine * H + 15) >> 4;      // tiles of the requests b0 .. b0 + ln
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int v = __shfl_up(upto, o, 64);
        if (ln >= o) upto += v;
      }
      const unsigned long long holds = __ballot(tile < upto);
      if (holds) {
        const int at = __ffsll((long long)holds) - 1;
        b = b0 + at;
        q_len = __shfl(mine, at, 64);
        tile -= at ? __shfl(upto, at - 1, 64) : 0;
      } else {
        tile -= __shfl(upto, 63, 64);
      }
    }
  }
  if (b < 0) return;   // (SOLO: this wave, and no barrier follows; else the whole workgroup: every wave counts the same)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, g = lane >> 4;
  const int DK = R + dr;
  const int start = seq_lens[b] - q_len;
  const int row0 = tile * 16;
  const int nrows = q_len * H - row0 < 16 ? q_len * H - row0 : 16;
  const bool rv = lr < nrows;
  const int tok = rv ? (row0 + lr) / H : 0, head = rv ? (row0 + lr) % H : 0;
  const int p = rv ? start + tok : -1;
  const int p_first = start + row0 / H, p_last = start + (row0 + nrows - 1) / H;
  const int first = window > 0 ? (p_first - window + 1 > 0 ? p_first - window + 1 : 0) : 0;
  const int lowest = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;   // of this lane's row
  const int kb0 = first & ~31;
  const int nblk = (p_last - kb0) / 32 + 1;
  const int parts = SOLO ? 1 : splits * 4, me = SOLO ? 0 : blockIdx.y * 4 + wave;
  const int per = (nblk + parts - 1) / parts;
  const int blk_lo = me * per, blk_hi = blk_lo + per < nblk ? blk_lo + per : nblk;
  const int32_t* bt = block_table + (int64_t)b * max_blocks;

  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
  bf16x8 qf[NC];
  {
    const bf16* qrow = qa + (int64_t)(cu_seqlens[b] + tok) * ld_qa + (int64_t)head * DK;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = 32 * c + 8 * g;
      qf[c] = (rv && d < DK) ? *(const bf16x8*)(qrow + d) : zero;
    }
  }
  f32x4 o[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // Row r of key tile t stands for key kb + 8 (r / 4) + 4 t + r % 4, so that the eight weights a lane holds after the
  // scores (rows 4g .. 4g+3 of both tiles) belong to the eight consecutive keys kb + 8g .. + 7: its operand of the
  // product with the values is 16 bytes of a transposed page.
  const int kofs = 8 * (lr >> 2) + (lr & 3);
  for (int blk = blk_lo; blk < blk_hi; ++blk) {
    const int kb = kb0 + blk * 32;
    const bf16* krow[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      int key = kb + kofs + 4 * t;
      key = key < first ? first : (key > p_last ? p_last : key);   // a row that exists; what lies outside is masked below
      krow[t] = cache + ((int64_t)bt[key / page] * page + (key % page)) * DK;
    }
    const bf16* vrow;
    {
      int key = kb + 8 * g;
      const int lo8 = first & ~7, hi8 = p_last & ~7;
      key = key < lo8 ? lo8 : (key > hi8 ? hi8 : key);
      vrow = cache_t + (int64_t)bt[key / page] * R * page + (key % page);
    }
    f32x4 s[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    // loads in groups, so that several are in flight before the first product waits
#pragma unroll
    for (int c0 = 0; c0 < NC; c0 += KG) {
      if (32 * c0 < DK) {
        bf16x8 ka[2][KG];
#pragma unroll
        for (int j = 0; j < KG; ++j) {
          // entries beyond the row meet zeros of the query; the address stays inside the row
          const int d = 32 * (c0 + j) + 8 * g;
          const int dc = d < DK ? d : 0;
#pragma unroll
          for (int t = 0; t < 2; ++t) ka[t][j] = *(const bf16x8*)(krow[t] + dc);
        }
#pragma unroll
        for (int j = 0; j < KG; ++j)
#pragma unroll
          for (int t = 0; t < 2; ++t)
            if (c0 + j < NC) s[t] = mfma16(ka[t][j], qf[c0 + j < NC ? c0 + j : 0], s[t]);
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = kb + 8 * g + 4 * t + i;
        const float v = (key <= p && key >= lowest) ? s[t][i] * scale_log2 : -INFINITY;
        s[t][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float alpha = m == -INFINITY ? 0.f : exp2_of(m - m_new);
    bf16x8 pb;
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = s[t][i] == -INFINITY ? 0.f : exp2_of(s[t][i] - m_new);
        psum += pv;
        pb[4 * t + i] = (bf16)pv;
      }
    l = l * alpha + psum;   // this lane's share of the row's sum; the four shares meet after the walk
    m = m_new;
#pragma unroll
    for (int t0 = 0; t0 < NT; t0 += VG) {
      if (16 * t0 < R) {
        bf16x8 va[VG];
#pragma unroll
        for (int j = 0; j < VG; ++j) {
          const int d = 16 * (t0 + j) + lr;
          va[j] = *(const bf16x8*)(vrow + (int64_t)(d < R ? d : 0) * page);
        }
#pragma unroll
        for (int j = 0; j < VG; ++j)
          if (t0 + j < NT && 16 * (t0 + j) < R) o[t0 + j] = mfma16(va[j], pb, o[t0 + j] * alpha);
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);

  // the waves meet: one after the other hands its state to wave 0
  const int ldm = R + 4;
  for (int w = 1; w < (SOLO ? 1 : 4); ++w) {
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (16 * t < R)
#pragma unroll
          for (int i = 0; i < 4; ++i) meet[lr * ldm + 16 * t + 4 * g + i] = o[t][i];
      if (g == 0) { meet[lr * ldm + R] = m; meet[lr * ldm + R + 1] = l; }
    }
    __syncthreads();
    if (wave == 0) {
      const float m2 = meet[lr * ldm + R], l2 = meet[lr * ldm + R + 1];
      const float mt = fmaxf(m, m2);
      const float a1 = m == -INFINITY ? 0.f : exp2_of(m - mt), a2 = m2 == -INFINITY ? 0.f : exp2_of(m2 - mt);
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (16 * t < R)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[t][i] = o[t][i] * a1 + meet[lr * ldm + 16 * t + 4 * g + i] * a2;
      l = l * a1 + l2 * a2;
      m = mt;
    }
    __syncthreads();
  }
  if ((!SOLO && wave != 0) || !rv) return;
  const int64_t trow = cu_seqlens[b] + tok;
  if (SOLO || splits == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16* orow = out + trow * ld_out + (int64_t)head * R;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (16 * t < R) {
        bf16x4 y;
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = (bf16)(o[t][i] * inv);
        *(bf16x4*)(orow + 16 * t + 4 * g) = y;
      }
  } else {
    float* pr = part + ((trow * H + head) * splits + blockIdx.y) * (int64_t)ldm;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (16 * t < R)
#pragma unroll
        for (int i = 0; i < 4; ++i) pr[16 * t + 4 * g + i] = o[t][i];
    if (g == 0) { pr[R] = m; pr[R + 1] = l; }
  }
}

// Steps with prompt portions, keys and values shared through LDS: the four waves of a workgroup take four consecutive row
// tiles of one request (64 rows) and walk the keys together; each block of 32 keys is brought into LDS once by the
// whole workgroup (its rows, and its latents transposed, both in 16-byte pieces) and every wave takes its MFMA operands
// from there, its queries too. The pieces of the next block are loaded into registers before a block is multiplied and
// written to LDS after it, so a block's trip to memory is hidden behind the block before. A wave whose rows lie before a
// block skips the arithmetic of that block, not the staging.
// FULL: R + dr is a multiple of 32, so no chunk of a row is cut short (no selects, LDS offsets known at compile time).
template <int NT, bool FULL>
__global__ void __launch_bounds__(256) latent_attn_lds_kernel(
    const bf16* __restrict__ qa, int64_t ld_qa, bf16* __restrict__ out, int64_t ld_out, const bf16* __restrict__ cache,
    const bf16* __restrict__ cache_t, const int32_t* __restrict__ block_table, int64_t max_blocks,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_lens, int num_reqs, float scale_log2,
    int window, int H, int R, int dr, int page, int page_shift) {
  constexpr int NC = NT / 2 + 4;
  constexpr int LDV = 40;              // a staged value row: 32 keys and 8 of padding
  extern __shared__ __attribute__((aligned(16))) bf16 stage[];
  const int DK = R + dr, LDK = DK + 8;
  bf16* Ks = stage;                    // [32][LDK]
  bf16* Vs = stage + 32 * LDK;         // [R][LDV]
  // which request and which of its groups of four row tiles; the last groups of a prompt walk the most keys and start
  // first, so that the short ones fill the gaps at the end
  int grp = (int)gridDim.x - 1 - (int)blockIdx.x, b = -1, q_len = 0;
  {
    const int ln = threadIdx.x & 63;
    for (int b0 = 0; b0 < num_reqs && b < 0; b0 += 64) {
      const int mine = b0 + ln < num_reqs ? cu_seqlens[b0 + ln + 1] - cu_seqlens[b0 + ln] : 0;
      int upto = (mine * H + 63) >> 6;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int v = __shfl_up(upto, o, 64);
        if (ln >= o) upto += v;
      }
      const unsigned long long holds = __ballot(grp < upto);
      if (holds) {
        const int at = __ffsll((long long)holds) - 1;
        b = b0 + at;
        q_len = __shfl(mine, at, 64);
        grp -= at ? __shfl(upto, at - 1, 64) : 0;
      } else {
        grp -= __shfl(upto, 63, 64);
      }
    }
  }
  if (b < 0) return;   // (the whole workgroup: every wave counts the same)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, g = lane >> 4;
  const int start = seq_lens[b] - q_len;
  const int all_rows = q_len * H;
  const int row0 = (grp * 4 + wave) * 16;
  const int nrows = all_rows - row0 < 16 ? all_rows - row0 : 16;   // <= 0: this wave has no rows, it only stages
  const bool rv = lr < nrows;
  const int tok = rv ? (row0 + lr) / H : 0, head = rv ? (row0 + lr) % H : 0;
  const int p = rv ? start + tok : -1;
  const int my_last = nrows > 0 ? start + (row0 + nrows - 1) / H : -1;
  const int w_pmin = start + row0 / H;     // the earliest position among the wave's rows
  // of the whole workgroup
  const int g_row0 = grp * 64;
  const int g_rows = all_rows - g_row0 < 64 ? all_rows - g_row0 : 64;
  const int p_first = start + g_row0 / H, p_last = start + (g_row0 + g_rows - 1) / H;
  const int first = window > 0 ? (p_first - window + 1 > 0 ? p_first - window + 1 : 0) : 0;
  const int lowest = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int kb0 = first & ~31;
  const int nblk = (p_last - kb0) / 32 + 1;
  const int32_t* bt = block_table + (int64_t)b * max_blocks;

  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
  const int kp = DK >> 3;                      // 16-byte pieces of a key row
  // this wave's queries wait in LDS (in registers they would leave no room for the next block's pieces)
  bf16* Qs = stage + 32 * LDK + R * LDV + wave * 16 * LDK;    // [16][LDK]
  for (int q = lane; q < 16 * kp; q += 64) {
    const int row = q / kp, pc = q - row * kp;
    bf16x8 v = zero;
    if (row < nrows) {
      const int r = row0 + row;
      v = *(const bf16x8*)(qa + (int64_t)(cu_seqlens[b] + r / H) * ld_qa + (int64_t)(r % H) * DK + pc * 8);
    }
    *(bf16x8*)(Qs + row * LDK + pc * 8) = v;
  }
  f32x4 o[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const int kofs = 8 * (lr >> 2) + (lr & 3);   // row of a key tile -> key, as in the kernel above
  const int lo8 = first & ~7, hi8 = p_last & ~7;
  // a thread's pieces of a block: of its rows (piece q is row q / kp, piece q % kp) and of its latents transposed
  // (piece q is latent entry q / 4, keys 8 (q % 4) .. + 7)
  constexpr int KP = (32 * (2 * NT + 16) + 255) / 256, VP = (64 * NT + 255) / 256;
  bf16x8 kn[KP], vn[VP];
  // piece q of the rows is row q / kp: the division is the high half of a multiplication by ceil(2^32 / kp), worked out
  // once (exact for the q < 32 kp and 2 <= kp < 300 that occur: R + dr is at least 16 and at most 640 here)
  const unsigned recip = (unsigned)((0x100000000ull + (unsigned)kp - 1u) / (unsigned)kp);
  const int pmask = page - 1;     // the page size is a power of two here
  const int page_lo = first >> page_shift, page_hi = p_last >> page_shift;
  auto fetch = [&](int kb) {
    // the block's pages (up to four where pages are shorter than a block): the same for every lane, so their table
    // entries and base offsets are scalar work; a page beyond the request's keys is replaced by its last one, whose
    // rows exist (what they hold is masked)
    int64_t pid[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int pg = ((kb + (j << page_shift)) >> page_shift);
      pg = pg < page_lo ? page_lo : (pg > page_hi ? page_hi : pg);
      pid[j] = __builtin_amdgcn_readfirstlane(bt[pg]);
    }
    const int kbm = kb & pmask;
#pragma unroll
    for (int u = 0; u < KP; ++u) {
      const int q = u * 256 + (int)threadIdx.x;
      if (q < 32 * kp) {
        const int row = (int)__umulhi((unsigned)q, recip), col = (q - row * kp) * 8;
        const int j = (kbm + row) >> page_shift;      // 0 .. 3 (0 where a page holds the whole block)
        const int64_t pg = j == 0 ? pid[0] : j == 1 ? pid[1] : j == 2 ? pid[2] : pid[3];
        kn[u] = *(const bf16x8*)(cache + ((pg << page_shift) + ((kbm + row) & pmask)) * DK + col);
      }
    }
#pragma unroll
    for (int u = 0; u < VP; ++u) {
      const int q = u * 256 + (int)threadIdx.x;
      if (q < 4 * R) {
        const int k8 = kbm + 8 * (q & 3);
        const int j = k8 >> page_shift;
        const int64_t pg = j == 0 ? pid[0] : j == 1 ? pid[1] : j == 2 ? pid[2] : pid[3];
        vn[u] = *(const bf16x8*)(cache_t + ((pg * R + (q >> 2)) << page_shift) + (k8 & pmask));
      }
    }
  };
  fetch(kb0);
  for (int blk = 0; blk < nblk; ++blk) {
    const int kb = kb0 + blk * 32;
    __syncthreads();   // the block before has been read
#pragma unroll
    for (int u = 0; u < KP; ++u) {
      const int q = u * 256 + (int)threadIdx.x;
      if (q < 32 * kp) {
        const int row = (int)__umulhi((unsigned)q, recip);
        *(bf16x8*)(Ks + row * LDK + (q - row * kp) * 8) = kn[u];
      }
    }
#pragma unroll
    for (int u = 0; u < VP; ++u) {
      const int q = u * 256 + (int)threadIdx.x;
      if (q < 4 * R) *(bf16x8*)(Vs + (q >> 2) * LDV + 8 * (q & 3)) = vn[u];
    }
    __syncthreads();
    if (blk + 1 < nblk) fetch(kb + 32);    // the next block's pieces travel while this one is multiplied
    if (kb > my_last) continue;    // (the wave: all its rows lie before this block; it still meets the barriers above)
    f32x4 s[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if (32 * c < DK) {
        if constexpr (FULL) {
          const bf16x8 qv = *(const bf16x8*)(Qs + lr * LDK + 8 * g + 32 * c);
#pragma unroll
          for (int t = 0; t < 2; ++t)
            s[t] = mfma16(*(const bf16x8*)(Ks + (kofs + 4 * t) * LDK + 8 * g + 32 * c), qv, s[t]);
        } else {
          const int d = 32 * c + 8 * g;
          const int dc = d < DK ? d : 0;     // entries beyond the row: the query's count as zeros
          bf16x8 qv = *(const bf16x8*)(Qs + lr * LDK + dc);
          if (d >= DK) qv = zero;
#pragma unroll
          for (int t = 0; t < 2; ++t)
            s[t] = mfma16(*(const bf16x8*)(Ks + (kofs + 4 * t) * LDK + dc), qv, s[t]);
        }
      }
    }
    float mx = -INFINITY;
    // a block that every row of the wave sees whole needs no mask (most blocks of a long prompt)
    const bool whole = nrows == 16 && kb + 31 <= w_pmin && (window == 0 || kb >= my_last - window + 1);
    if (whole) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[t][i] *= scale_log2;
          mx = fmaxf(mx, s[t][i]);
        }
    } else {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb + 8 * g + 4 * t + i;
          const float v = (key <= p && key >= lowest) ? s[t][i] * scale_log2 : -INFINITY;
          s[t][i] = v;
          mx = fmaxf(mx, v);
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // The running maximum follows the scores only when one of the wave's rows has outgrown it by more than 2^8 (or has
    // none yet): the weights may then exceed 1, up to 256, which float sums and bf16 weights hold without loss, and
    // the 4 x NT multiplications that bring the output to a new maximum are done on few blocks instead of on all.
    if (__any(mx > m + 8.f)) {
      const float m_new = fmaxf(m, mx);
      const float alpha = m == -INFINITY ? 0.f : exp2_of(m - m_new);
      l *= alpha;
      m = m_new;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        if (16 * t < R) o[t] = o[t] * alpha;
    }
    bf16x8 pb;
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = s[t][i] == -INFINITY ? 0.f : exp2_of(s[t][i] - m);
        psum += pv;
        pb[4 * t + i] = (bf16)pv;
      }
    l += psum;
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (16 * t < R) o[t] = mfma16(*(const bf16x8*)(Vs + (16 * t + lr) * LDV + 8 * g), pb, o[t]);
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!rv) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  bf16* orow = out + (int64_t)(cu_seqlens[b] + tok) * ld_out + (int64_t)head * R;
#pragma unroll
  for (int t = 0; t < NT; ++t)
    if (16 * t < R) {
      bf16x4 y;
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = (bf16)(o[t][i] * inv);
      *(bf16x4*)(orow + 16 * t + 4 * g) = y;
    }
}

// One workgroup per (token, head) row: the parts' (max, sum, output) become the row's output. A part is R + 4 floats
// (output, max, sum, two unused), so its rows are read 16 bytes a lane.
__global__ void __launch_bounds__(128) latent_attn_merge_kernel(const float* __restrict__ part, bf16* __restrict__ out,
                                                                int64_t ld_out, int H, int R, int splits) {
  __shared__ float wgt[256];
  __shared__ float inv_s;
  const int64_t row = blockIdx.x;
  const int ldm = R + 4;
  const float* pr = part + row * splits * (int64_t)ldm;
  if (threadIdx.x < 64) {     // the first wave: the weights of the parts
    float mt = -INFINITY;
    for (int s = threadIdx.x; s < splits; s += 64) mt = fmaxf(mt, pr[s * (int64_t)ldm + R]);
    mt = wave_max(mt);
    float lt = 0.f;
    for (int s = threadIdx.x; s < splits; s += 64) {
      const float ms = pr[s * (int64_t)ldm + R];
      const float w = ms == -INFINITY ? 0.f : exp2_of(ms - mt);
      wgt[s] = w;
      lt += w * pr[s * (int64_t)ldm + R + 1];
    }
    lt = wave_sum(lt);
    if (threadIdx.x == 0) inv_s = lt > 0.f ? 1.f / lt : 0.f;
  }
  __syncthreads();
  const float inv = inv_s;
  bf16* orow = out + (row / H) * ld_out + (row % H) * (int64_t)R;
  for (int d = threadIdx.x * 4; d < R; d += 128 * 4) {
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < splits; ++s) {
      const f32x4 v = *(const f32x4*)(pr + s * (int64_t)ldm + d);
      const float w = wgt[s];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(w, v[i], acc[i]);
    }
    bf16x4 y;
#pragma unroll
    for (int i = 0; i < 4; ++i) y[i] = (bf16)(acc[i] * inv);
    *(bf16x4*)(orow + d) = y;
  }
}

}  // namespace

// proj [T, ld]: the queries at column q_off (head h at h*(dn+dr): dn unrotated, then dr rotated), the down projection
// at c_off (R latent, then dr shared key part; c_off < 0: this layer has none and nothing is written to the cache).
// cos_sin [positions, rot] = [cos | sin] of rot/2 angles (null: no rotation); the first `rot` entries of a rotated part
// turn. qa [T, ld_qa]: head h at h*(R+dr); its last dr entries are written here. cache [blocks*page, R+dr].
// style: 1 pairs (2i, 2i+1), 0 pairs (i, i + rot/2). q_src (may be null: the queries are in proj): [T, ld_qs], the
// queries at column q_off of it.
extern "C" int dinfer_latent_post(int dtype, const void* proj, int64_t tokens, int64_t ld, int q_off, int c_off, int heads,
                                  int dn, int dr, int R, const void* gain, int w_f32, float eps,
                                  const int32_t* positions, const float* cos_sin, int rot, void* qa, int64_t ld_qa,
                                  void* cache, void* cache_t, int page_size, const int64_t* slots, int style,
                                  const void* q_src, int64_t ld_qs, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (style != 0 && style != 1) return ERR_UNSUPPORTED;
  if (heads <= 0 || dn < 0 || dr < 0 || R <= 0 || rot < 0 || rot > dr || (rot & 1) || tokens > 0x7fffffff ||
      ld_qa < (int64_t)heads * (R + dr) || (cache_t && page_size <= 0))
    return ERR_BAD_SHAPE;
  DINFER_DISPATCH_DTYPE(dtype, {
    latent_post_kernel<S><<<(unsigned)tokens, 256, 0, stream>>>((const S*)proj, ld, q_off, c_off, heads, dn, dr, R, gain,
                                                               w_f32, eps, positions, cos_sin, rot, (S*)qa, ld_qa,
                                                               (S*)cache, (S*)cache_t, page_size, slots, style,
                                                               (const S*)q_src, ld_qs);
  });
  return launch_status();
}

extern "C" int dinfer_latent_attn_ref(int dtype, const void* qa, int64_t ld_qa, void* out, int64_t ld_out,
                                      const void* cache, const int32_t* block_table, int64_t max_blocks,
                                      const int32_t* cu_seqlens, const int32_t* seq_lens, int num_reqs, int64_t tokens,
                                      float scale, int window, int heads, int R, int dr, int page_size,
                                      hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (heads <= 0 || R <= 0 || dr < 0 || page_size <= 0 || max_blocks <= 0 || window < 0 || tokens > 0x7fffffff)
    return ERR_BAD_SHAPE;
  if (R > MAX_R || R + dr > MAX_DK) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((heads + WAVES - 1) / WAVES));
  const size_t lds = (size_t)WAVES * (R + dr + 64) * sizeof(float);
  DINFER_DISPATCH_DTYPE(dtype, {
    latent_attn_ref_kernel<S><<<grid, WAVES * 64, lds, stream>>>((const S*)qa, ld_qa, (S*)out, ld_out, (const S*)cache,
                                                                 block_table, max_blocks, cu_seqlens, seq_lens,
                                                                 num_reqs, scale, window, heads, R, dr, page_size);
  });
  return launch_status();
}

// Whether latent_attn_mfma takes these sizes.
extern "C" int dinfer_latent_mfma_supports(int R, int dr, int page_size) {
  return R >= 16 && R <= 512 && R % 16 == 0 && dr >= 0 && dr <= 128 && dr % 8 == 0 && page_size > 0 && page_size % 8 == 0;
}

// bf16. cache [blocks, page, R + dr] and cache_t [blocks, R, page]. splits > 1: every request brings one row; part holds
// tokens * heads * splits * (R + 4) floats.
extern "C" int dinfer_latent_attn_mfma(const void* qa, int64_t ld_qa, void* out, int64_t ld_out, float* part,
                                       int64_t part_floats, const void* cache, const void* cache_t,
                                       const int32_t* block_table, int64_t max_blocks, const int32_t* cu_seqlens,
                                       const int32_t* seq_lens, int num_reqs, int64_t tokens, float scale, int window,
                                       int heads, int R, int dr, int page_size, int splits, hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (heads <= 0 || max_blocks <= 0 || window < 0 || tokens > 0x7fffffff || splits < 1 || ld_qa % 8 || ld_out % 4 ||
      ((uintptr_t)qa % 16) || ((uintptr_t)out % 8) || ((uintptr_t)cache % 16) || ((uintptr_t)cache_t % 16))
    return ERR_BAD_SHAPE;
  if (!dinfer_latent_mfma_supports(R, dr, page_size)) return ERR_UNSUPPORTED;
  if (splits > 1 && (tokens != num_reqs || !part || part_floats < tokens * heads * splits * (int64_t)(R + 4) || splits > 256))
    return ERR_WORKSPACE;
  const int64_t tiles = (tokens * heads + 15) / 16 + num_reqs;
  if (tiles > 0x7fffffff || splits > 65535) return ERR_UNSUPPORTED;
  const bool solo = tokens != num_reqs;      // some request brings more than one row
  // keys, 4 x 16 queries and values of a block in LDS: where that fits (and pages are a power of two) prompt portions
  // take the kernel that shares them; else every wave walks its own keys
  const size_t bytes = ((size_t)(32 + 64) * (R + dr + 8) + (size_t)R * 40) * sizeof(bf16);
  constexpr size_t LDS_MOST = 160 * 1024 - 1024;
  if (solo && (page_size & (page_size - 1)) == 0 && bytes <= LDS_MOST) {
    const int page_shift = __builtin_ctz(page_size);
    const int64_t groups = (tokens * heads + 63) / 64 + num_reqs;
    if (groups > 0x7fffffff) return ERR_UNSUPPORTED;
    const float sl2 = scale * LOG2E;
#define LDS_LAUNCH_(NT, FULL)                                                                                                 \
  do {                                                                                                                 \
    static bool sized = false;                                                                                         \
    if (!sized) {                                                                                                      \
      if (hipFuncSetAttribute((const void*)latent_attn_lds_kernel<NT, FULL>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                              (int)LDS_MOST) != hipSuccess)                                                             \
        return ERR_LAUNCH;                                                                                             \
      sized = true;                                                                                                    \
    }                                                                                                                  \
    latent_attn_lds_kernel<NT, FULL><<<(unsigned)groups, 256, bytes, stream>>>(                                        \
        (const bf16*)qa, ld_qa, (bf16*)out, ld_out, (const bf16*)cache, (const bf16*)cache_t, block_table, max_blocks, \
        cu_seqlens, seq_lens, num_reqs, sl2, window, heads, R, dr, page_size, page_shift);                                      \
  } while (0)
#define LDS_LAUNCH(NT) do { if ((R + dr) % 32 == 0) LDS_LAUNCH_(NT, true); else LDS_LAUNCH_(NT, false); } while (0)
    if (R <= 64) LDS_LAUNCH(4);
    else if (R <= 128) LDS_LAUNCH(8);
    else if (R <= 256) LDS_LAUNCH(16);
    else LDS_LAUNCH(32);
#undef LDS_LAUNCH
#undef LDS_LAUNCH_
    return launch_status();
  }
  const dim3 grid((unsigned)(solo ? (tiles + 3) / 4 : tiles), (unsigned)(solo ? 1 : splits));
  const size_t lds = solo ? 0 : (size_t)16 * (R + 4) * sizeof(float);
  const float sl = scale * LOG2E;
#define LAUNCH(NT, SOLO)                                                                                               \
  latent_attn_mfma_kernel<NT, SOLO><<<grid, 256, lds, stream>>>(                                                       \
      (const bf16*)qa, ld_qa, (bf16*)out, ld_out, part, (const bf16*)cache, (const bf16*)cache_t, block_table,        \
      max_blocks, cu_seqlens, seq_lens, num_reqs, sl, window, heads, R, dr, page_size, solo ? 1 : splits)
#define PICK(NT) do { if (solo) LAUNCH(NT, true); else LAUNCH(NT, false); } while (0)
  if (R <= 64) PICK(4);
  else if (R <= 128) PICK(8);
  else if (R <= 256) PICK(16);
  else PICK(32);
#undef PICK
#undef LAUNCH
  if (solo) return launch_status();
  if (launch_status() != OK) return ERR_LAUNCH;
  if (splits > 1)
    latent_attn_merge_kernel<<<(unsigned)(tokens * heads), 128, 0, stream>>>(part, (bf16*)out, ld_out, heads, R, splits);
  return launch_status();
}
