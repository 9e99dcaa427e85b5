// Embedding row gather, gated activation (SwiGLU), residual add and dtype
// widening. All of them are memory-bound; rows are moved in 16-byte pieces
// when sizes and pointers allow it.
//
// Reference behaviour: crates/kernels/cuda/activation.cu:8-16,80-99,121-129
// (silu(x) = x / (1 + exp(-x)), an id outside [0, vocab) reads row 0) and
// crates/kernels/cuda/elementwise.cu:42-46 (add in float, one rounding).
#include "common.cuh"

using namespace dinfer;

namespace {

template <class S>
__global__ void __launch_bounds__(256) embedding_kernel(const int32_t* __restrict__ ids, const S* __restrict__ table,
                                                        S* __restrict__ out, int64_t vocab, int64_t width, int vec_ok,
                                                        const int32_t* __restrict__ from,
                                                        const int32_t* __restrict__ last) {
  const int64_t t = blockIdx.x;
  // from[t] >= 0: the token is not known to the host yet, it is that one of the tokens the step before sampled
  int64_t id = ids[t];
  if (from) {
    const int32_t at = from[t];
    if (at >= 0) id = last[at];
  }
  if (id < 0 || id >= vocab) id = 0;
  const S* src = table + id * width;
  S* dst = out + t * width;
  if (vec_ok) {
    const int64_t n16 = width * (int64_t)sizeof(S) / 16;
    const uint4* s4 = (const uint4*)src;
    uint4* d4 = (uint4*)dst;
    for (int64_t i = threadIdx.x; i < n16; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int64_t i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
  }
}

__device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }

// in [T, 2*inter] with row stride ld_in: gate = cols [0, inter), up = cols [inter, 2*inter).
template <class S>
__global__ void __launch_bounds__(256) swiglu_kernel(const S* __restrict__ in, S* __restrict__ out, int64_t inter,
                                                     int64_t ld_in) {
  const int64_t t = blockIdx.y;
  const S* g = in + t * ld_in;
  const S* u = g + inter;
  S* o = out + t * inter;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < inter; i += (int64_t)gridDim.x * blockDim.x)
    o[i] = from_f32<S>(silu(to_f32(g[i])) * to_f32(u[i]));
}

// 8 bf16 per thread and iteration; needs inter % 8 == 0 and 16-byte aligned rows.
__global__ void __launch_bounds__(256) swiglu_bf16x8_kernel(const bf16* __restrict__ in, bf16* __restrict__ out,
                                                            int64_t inter, int64_t ld_in) {
  const int64_t t = blockIdx.y;
  const bf16x8* g = (const bf16x8*)(in + t * ld_in);
  const bf16x8* u = (const bf16x8*)(in + t * ld_in + inter);
  bf16x8* o = (bf16x8*)(out + t * inter);
  const int64_t n8 = inter / 8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    const bf16x8 gv = g[i], uv = u[i];
    bf16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (bf16)(silu((float)gv[j]) * (float)uv[j]);
    o[i] = r;
  }
}

// dst[i] = round(float(dst[i]) + float(src[i]))
template <class S>
__global__ void __launch_bounds__(256) add_inplace_kernel(S* __restrict__ dst, const S* __restrict__ src, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = from_f32<S>(to_f32(dst[i]) + to_f32(src[i]));
}

template <class S>
__global__ void __launch_bounds__(256) widen_kernel(const S* __restrict__ src, float* __restrict__ dst, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = to_f32(src[i]);
}

// x[r][c] = cap * tanh(x[r][c] * scale / cap) (cap <= 0: x * scale), in place, rows of `width` at stride ld
template <class S>
__global__ void __launch_bounds__(256) scale_softcap_kernel(S* __restrict__ x, int64_t ld, int64_t width, float scale,
                                                            float cap) {
  S* row = x + (int64_t)blockIdx.y * ld;
  const float inv = cap > 0.f ? 1.f / cap : 0.f;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < width; i += (int64_t)gridDim.x * blockDim.x) {
    float v = to_f32(row[i]) * scale;
    if (cap > 0.f) v = cap * tanhf(v * inv);
    row[i] = from_f32<S>(v);
  }
}

// Fills n 32-bit words; used where a captured graph must not hold a memset node.
__global__ void __launch_bounds__(256) fill_u32_kernel(uint32_t* __restrict__ dst, uint32_t v, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = v;
}

inline unsigned blocks_for(int64_t n, int per_block, unsigned cap) {
  int64_t b = (n + per_block - 1) / per_block;
  if (b < 1) b = 1;
  return (unsigned)(b > cap ? cap : b);
}

// out[t] = table[id] * scale with types of their own: a bf16 table may feed a float residual stream.
template <class S, class O>
__global__ void __launch_bounds__(256) embedding_to_kernel(const int32_t* __restrict__ ids, const S* __restrict__ table,
                                                           O* __restrict__ out, int64_t vocab, int64_t width, float scale,
                                                           const int32_t* __restrict__ from,
                                                           const int32_t* __restrict__ last) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  if (from) {
    const int32_t at = from[t];
    if (at >= 0) id = last[at];
  }
  if (id < 0 || id >= vocab) id = 0;
  const S* src = table + id * width;
  O* dst = out + t * width;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_f32<O>(to_f32(src[i]) * scale);
}

// Activations of one argument: 0 silu, 1 the square of relu, 2 gelu in its tanh form, 3 gelu with the error function,
// 4 the logistic function, 5 the hyperbolic tangent.
__device__ __forceinline__ float act1(float z, int act) {
  if (act == 5) return tanhf(z);
  if (act == 0) return z / (1.f + expf(-z));
  if (act == 1) { const float r = fmaxf(z, 0.f); return r * r; }
  if (act == 3) return 0.5f * z * (1.f + erff(z * 0.7071067811865476f));
  if (act == 4) return 1.f / (1.f + expf(-z));
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <class S>
__global__ void __launch_bounds__(256) act_kernel(const S* __restrict__ in, int64_t ld_in, S* __restrict__ out,
                                                  int64_t ld_out, int64_t n, int act) {
  const int64_t t = blockIdx.y;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[t * ld_out + i] = from_f32<S>(act1(to_f32(in[t * ld_in + i]), act));
}

// entry i of x meets entry i / group of g: one gate for every `group` consecutive columns (a head), group 1: one each
template <class S>
__global__ void __launch_bounds__(256) gate_kernel(S* __restrict__ x, int64_t ld_x, const S* __restrict__ g, int64_t ld_g,
                                                   int64_t n, int act, int64_t group) {
  const int64_t t = blockIdx.y;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    x[t * ld_x + i] = from_f32<S>(to_f32(x[t * ld_x + i]) * act1(to_f32(g[t * ld_g + (group > 1 ? i / group : i)]), act));
}

// out[t, i] = act(in[t, i]) * in[t, inter + i] for any activation of act1
template <class S>
__global__ void __launch_bounds__(256) gated_any_kernel(const S* __restrict__ in, S* __restrict__ out, int64_t inter,
                                                        int64_t ld_in, int act) {
  const int64_t t = blockIdx.y;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < inter; i += (int64_t)gridDim.x * blockDim.x)
    out[t * inter + i] = from_f32<S>(act1(to_f32(in[t * ld_in + i]), act) * to_f32(in[t * ld_in + inter + i]));
}

// The same, 8 bf16 per thread and iteration; needs inter % 8 == 0 and 16-byte aligned rows.
__global__ void __launch_bounds__(256) gated_any_bf16x8_kernel(const bf16* __restrict__ in, bf16* __restrict__ out,
                                                               int64_t inter, int64_t ld_in, int act) {
  const int64_t t = blockIdx.y;
  const bf16x8* g = (const bf16x8*)(in + t * ld_in);
  const bf16x8* u = (const bf16x8*)(in + t * ld_in + inter);
  bf16x8* o = (bf16x8*)(out + t * inter);
  const int64_t n8 = inter / 8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    const bf16x8 gv = g[i], uv = u[i];
    bf16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (bf16)(act1((float)gv[j], act) * (float)uv[j]);
    o[i] = r;
  }
}

// Token shift: out[t] = x[t] + (before - x[t]) * mix, `before` the row of the token before in its request: the row
// above inside a step's portion, the request's kept row (state[slot]) for a portion's first row. The thread that
// serves a portion's first row then keeps the portion's last row for the next step, so nobody reads the kept row
// after it has been replaced. A workgroup takes one request and TOK of its rows.
constexpr int SHIFT_TOK = 8;
template <class S>
__global__ void __launch_bounds__(256) token_shift_kernel(const S* __restrict__ x, int64_t ld_x, S* __restrict__ out,
                                                          int64_t ld_out, S* __restrict__ state,
                                                          const float* __restrict__ mix, const int32_t* __restrict__ cu,
                                                          const int32_t* __restrict__ seq_lens,
                                                          const int32_t* __restrict__ slots, int64_t width) {
  const int b = blockIdx.y;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  const bool starts = seq_lens[b] - n <= 0;   // the request's first token: zeros before it, whatever the slot held
  const int r0 = blockIdx.x * SHIFT_TOK;
  if (r0 >= n) return;
  const int r1 = r0 + SHIFT_TOK < n ? r0 + SHIFT_TOK : n;
  S* kept = state + (int64_t)slots[b] * width;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    const float m = mix[i];
    float before = r0 > 0 ? to_f32(x[(int64_t)(t0 + r0 - 1) * ld_x + i]) : starts ? 0.f : to_f32(kept[i]);
    for (int r = r0; r < r1; ++r) {
      const float v = to_f32(x[(int64_t)(t0 + r) * ld_x + i]);
      out[(int64_t)(t0 + r) * ld_out + i] = from_f32<S>(v + (before - v) * m);
      before = v;
    }
    if (r0 == 0) kept[i] = x[(int64_t)(t0 + n - 1) * ld_x + i];
  }
}

}  // namespace

// src, last (both or neither): where src[t] >= 0, token t's id is last[src[t]] instead of ids[t].
extern "C" int dinfer_embedding(int dtype, const int32_t* ids, const void* table, void* out, int64_t tokens,
                                int64_t vocab, int64_t width, const int32_t* src, const int32_t* last,
                                hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (vocab <= 0 || width <= 0 || tokens > 0x7fffffff || (!src != !last)) return ERR_BAD_SHAPE;
  DINFER_DISPATCH_DTYPE(dtype, {
    const bool vec = (width * sizeof(S)) % 16 == 0 && ((uintptr_t)table % 16 == 0) && ((uintptr_t)out % 16 == 0);
    embedding_kernel<S><<<(unsigned)tokens, 256, 0, stream>>>(ids, (const S*)table, (S*)out, vocab, width, vec ? 1 : 0,
                                                              src, last);
  });
  return launch_status();
}

// act: 0 = silu, 2 = gelu in its tanh form (the codes of act1). Anything else is refused.
extern "C" int dinfer_gated_act(int dtype, int act, const void* in, void* out, int64_t tokens, int64_t inter,
                                int64_t ld_in, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (act != 0 && act != 2) return ERR_UNSUPPORTED;
  if (inter <= 0 || ld_in < 2 * inter || tokens > 65535 * 1024LL) return ERR_BAD_SHAPE;
  if (act != 0) {
    for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
      const int64_t nt = tokens - t0 < 65535 ? tokens - t0 : 65535;
      const dim3 grid(blocks_for(inter, 256, 64), (unsigned)nt);
      if (dtype == DT_BF16 && inter % 8 == 0 && ld_in % 8 == 0 && ((uintptr_t)in % 16 == 0) && ((uintptr_t)out % 16 == 0)) {
        gated_any_bf16x8_kernel<<<dim3(blocks_for(inter / 8, 256, 64), (unsigned)nt), 256, 0, stream>>>(
            (const bf16*)in + t0 * ld_in, (bf16*)out + t0 * inter, inter, ld_in, act);
        continue;
      }
      DINFER_DISPATCH_DTYPE(dtype, {
        gated_any_kernel<S><<<grid, 256, 0, stream>>>((const S*)in + t0 * ld_in, (S*)out + t0 * inter, inter, ld_in, act);
      });
    }
    return launch_status();
  }
  // grid.y is limited to 65535 rows; larger batches are cut into slabs
  for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
    const int64_t nt = tokens - t0 < 65535 ? tokens - t0 : 65535;
    if (dtype == DT_BF16) {
      const bf16* ip = (const bf16*)in + t0 * ld_in;
      bf16* op = (bf16*)out + t0 * inter;
      const bool vec = inter % 8 == 0 && ld_in % 8 == 0 && ((uintptr_t)ip % 16 == 0) && ((uintptr_t)op % 16 == 0);
      if (vec)
        swiglu_bf16x8_kernel<<<dim3(blocks_for(inter / 8, 256, 64), (unsigned)nt), 256, 0, stream>>>(ip, op, inter, ld_in);
      else
        swiglu_kernel<bf16><<<dim3(blocks_for(inter, 256, 64), (unsigned)nt), 256, 0, stream>>>(ip, op, inter, ld_in);
    } else if (dtype == DT_F32) {
      swiglu_kernel<float><<<dim3(blocks_for(inter, 256, 64), (unsigned)nt), 256, 0, stream>>>(
          (const float*)in + t0 * ld_in, (float*)out + t0 * inter, inter, ld_in);
    } else {
      return ERR_BAD_DTYPE;
    }
  }
  return launch_status();
}

// x[:rows, :width] (row stride ld) *= scale, then softly capped at +-cap (cap * tanh(x / cap); cap <= 0: no cap).
extern "C" int dinfer_scale_softcap(int dtype, void* x, int64_t ld, int64_t rows, int64_t width, float scale, float cap,
                                    hipStream_t stream) {
  if (rows <= 0 || width <= 0) return OK;
  if (ld < width || rows > 65535) return ERR_BAD_SHAPE;
  DINFER_DISPATCH_DTYPE(dtype, {
    scale_softcap_kernel<S><<<dim3(blocks_for(width, 256, 256), (unsigned)rows), 256, 0, stream>>>((S*)x, ld, width, scale, cap);
  });
  return launch_status();
}

extern "C" int dinfer_add_inplace(int dtype, void* dst, const void* src, int64_t n, hipStream_t stream) {
  if (n <= 0) return OK;
  DINFER_DISPATCH_DTYPE(dtype, {
    add_inplace_kernel<S><<<blocks_for(n, 256, 4096), 256, 0, stream>>>((S*)dst, (const S*)src, n);
  });
  return launch_status();
}

extern "C" int dinfer_widen(int dtype, const void* src, float* dst, int64_t n, hipStream_t stream) {
  if (n <= 0) return OK;
  DINFER_DISPATCH_DTYPE(dtype, {
    widen_kernel<S><<<blocks_for(n, 256, 4096), 256, 0, stream>>>((const S*)src, dst, n);
  });
  return launch_status();
}

extern "C" int dinfer_fill_u32(void* dst, uint32_t value, int64_t n_words, hipStream_t stream) {
  if (n_words <= 0) return OK;
  fill_u32_kernel<<<blocks_for(n_words, 256, 4096), 256, 0, stream>>>((uint32_t*)dst, value, n_words);
  return launch_status();
}

extern "C" int dinfer_embedding_to(int table_dtype, int out_dtype, const int32_t* ids, const void* table, void* out,
                                   int64_t tokens, int64_t vocab, int64_t width, float scale, const int32_t* src,
                                   const int32_t* last, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (vocab <= 0 || width <= 0 || tokens > 0x7fffffff || (!src != !last)) return ERR_BAD_SHAPE;
  const unsigned g = (unsigned)tokens;
  if (table_dtype == DT_BF16 && out_dtype == DT_F32)
    embedding_to_kernel<bf16, float><<<g, 256, 0, stream>>>(ids, (const bf16*)table, (float*)out, vocab, width, scale, src, last);
  else if (table_dtype == DT_BF16 && out_dtype == DT_BF16)
    embedding_to_kernel<bf16, bf16><<<g, 256, 0, stream>>>(ids, (const bf16*)table, (bf16*)out, vocab, width, scale, src, last);
  else if (table_dtype == DT_F32 && out_dtype == DT_F32)
    embedding_to_kernel<float, float><<<g, 256, 0, stream>>>(ids, (const float*)table, (float*)out, vocab, width, scale, src, last);
  else
    return ERR_BAD_DTYPE;
  return launch_status();
}

// x[t, i] *= act(g[t, i]) for i < n: a gate on a block of columns (x and g point at the first column of theirs).
// group > 1: one gate for every `group` consecutive columns of x (g has n / group columns).
extern "C" int dinfer_gate(int dtype, int act, void* x, int64_t ld_x, const void* g, int64_t ld_g, int64_t tokens,
                           int64_t n, int64_t group, hipStream_t stream) {
  if (tokens <= 0 || n <= 0) return OK;
  if (act < 0 || act > 4) return ERR_UNSUPPORTED;
  if (group < 1 || n % group || ld_x < n || ld_g < n / group) return ERR_BAD_SHAPE;
  for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
    const int64_t nt = tokens - t0 < 65535 ? tokens - t0 : 65535;
    const dim3 grid((unsigned)((n + 1023) / 1024 < 64 ? (n + 1023) / 1024 : 64), (unsigned)nt);
    DINFER_DISPATCH_DTYPE(dtype, {
      gate_kernel<S><<<grid, 256, 0, stream>>>((S*)x + t0 * ld_x, ld_x, (const S*)g + t0 * ld_g, ld_g, n, act, group);
    });
  }
  return launch_status();
}

// out[t, i] = act(in[t, i]) for i < n (in place allowed). act: 0 silu, 1 relu squared, 2 gelu (tanh form), 3 gelu
// (error function), 4 logistic.
extern "C" int dinfer_act(int dtype, int act, const void* in, int64_t ld_in, void* out, int64_t ld_out, int64_t tokens,
                          int64_t n, hipStream_t stream) {
  if (tokens <= 0 || n <= 0) return OK;
  if (act < 0 || act > 5) return ERR_UNSUPPORTED;
  if (ld_in < n || ld_out < n) return ERR_BAD_SHAPE;
  for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
    const int64_t nt = tokens - t0 < 65535 ? tokens - t0 : 65535;
    const dim3 grid((unsigned)((n + 1023) / 1024 < 64 ? (n + 1023) / 1024 : 64), (unsigned)nt);
    DINFER_DISPATCH_DTYPE(dtype, {
      act_kernel<S><<<grid, 256, 0, stream>>>((const S*)in + t0 * ld_in, ld_in, (S*)out + t0 * ld_out, ld_out, n, act);
    });
  }
  return launch_status();
}

namespace {
// The same with 8 bf16 a thread (16-byte loads and stores): width % 8 == 0, rows and state 16-byte aligned. A thread
// keeps its 8 channels' shares and walks the workgroup's rows; grid.z cuts the width where a workgroup does not span it.
__global__ void __launch_bounds__(256) token_shift_bf16x8_kernel(const bf16* __restrict__ x, int64_t ld_x,
                                                                 bf16* __restrict__ out, int64_t ld_out,
                                                                 bf16* __restrict__ state, const float* __restrict__ mix,
                                                                 const int32_t* __restrict__ cu,
                                                                 const int32_t* __restrict__ seq_lens,
                                                                 const int32_t* __restrict__ slots, int64_t width) {
  const int b = blockIdx.y;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  const int r0 = blockIdx.x * SHIFT_TOK;
  const int64_t i = ((int64_t)blockIdx.z * blockDim.x + threadIdx.x) * 8;
  if (r0 >= n || i >= width) return;
  const bool starts = seq_lens[b] - n <= 0;
  const int r1 = r0 + SHIFT_TOK < n ? r0 + SHIFT_TOK : n;
  bf16* kept = state + (int64_t)slots[b] * width + i;
  const f32x4 m0 = *(const f32x4*)(mix + i), m1 = *(const f32x4*)(mix + i + 4);
  float m[8] = {m0[0], m0[1], m0[2], m0[3], m1[0], m1[1], m1[2], m1[3]};
  bf16x8 before;
  if (r0 > 0) before = *(const bf16x8*)(x + (int64_t)(t0 + r0 - 1) * ld_x + i);
  else if (starts) {
#pragma unroll
    for (int j = 0; j < 8; ++j) before[j] = (bf16)0.f;
  } else before = *(const bf16x8*)kept;
  // all rows' loads first: they do not depend on each other
  bf16x8 rows[SHIFT_TOK];
#pragma unroll
  for (int r = 0; r < SHIFT_TOK; ++r)
    if (r0 + r < r1) rows[r] = *(const bf16x8*)(x + (int64_t)(t0 + r0 + r) * ld_x + i);
#pragma unroll
  for (int r = 0; r < SHIFT_TOK; ++r) {
    if (r0 + r >= r1) break;
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = (float)rows[r][j];
      o[j] = (bf16)(v + ((float)before[j] - v) * m[j]);
    }
    *(bf16x8*)(out + (int64_t)(t0 + r0 + r) * ld_out + i) = o;
    before = rows[r];
  }
  if (r0 == 0) *(bf16x8*)kept = *(const bf16x8*)(x + (int64_t)(t0 + n - 1) * ld_x + i);
}
}  // namespace

// out[t] = x[t] + (row before - x[t]) * mix for the rows of num_reqs requests (cu_seqlens), the row before a
// portion's first row taken from state[slots[b]] (zeros for a request that starts), which then takes the portion's
// last row of x. x, out and state in the step's dtype, mix float [width]; out must not be x. max_rows: the longest
// portion of the step (or more). seq_lens: the requests' lengths after the step.
extern "C" int dinfer_token_shift(int dtype, const void* x, int64_t ld_x, void* out, int64_t ld_out, void* state,
                                  const float* mix, const int32_t* cu_seqlens, const int32_t* seq_lens,
                                  const int32_t* slots, int num_reqs,
                                  int64_t max_rows, int64_t width, hipStream_t stream) {
  if (num_reqs <= 0 || max_rows <= 0) return OK;
  if (width <= 0 || ld_x < width || ld_out < width || num_reqs > 65535 || x == out) return ERR_BAD_SHAPE;
  const dim3 grid((unsigned)((max_rows + SHIFT_TOK - 1) / SHIFT_TOK), (unsigned)num_reqs);
  if (dtype == DT_BF16 && width % 8 == 0 && ld_x % 8 == 0 && ld_out % 8 == 0 && ((uintptr_t)x % 16 == 0) &&
      ((uintptr_t)out % 16 == 0) && ((uintptr_t)state % 16 == 0) && ((uintptr_t)mix % 16 == 0)) {
    const int threads = width >= 2048 ? 256 : width >= 512 ? 64 * (int)((width / 8 + 63) / 64) : 64;
    const dim3 vgrid(grid.x, grid.y, (unsigned)((width / 8 + threads - 1) / threads));
    token_shift_bf16x8_kernel<<<vgrid, threads, 0, stream>>>((const bf16*)x, ld_x, (bf16*)out, ld_out, (bf16*)state, mix,
                                                             cu_seqlens, seq_lens, slots, width);
    return launch_status();
  }
  DINFER_DISPATCH_DTYPE(dtype, {
    token_shift_kernel<S><<<grid, width >= 256 ? 256 : 64, 0, stream>>>((const S*)x, ld_x, (S*)out, ld_out, (S*)state, mix,
                                                                        cu_seqlens, seq_lens, slots, width);
  });
  return launch_status();
}

namespace {

template <class S>
__global__ void __launch_bounds__(256) axpby_kernel(const S* __restrict__ a, int64_t ld_a, float alpha,
                                                    const S* __restrict__ b, int64_t ld_b, float beta,
                                                    S* __restrict__ out, int64_t ld_out, int64_t cols) {
  const int64_t t = blockIdx.y;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < cols; i += (int64_t)gridDim.x * blockDim.x)
    out[t * ld_out + i] = from_f32<S>(alpha * to_f32(a[t * ld_a + i]) + beta * to_f32(b[t * ld_b + i]));
}

template <class SX, class SA, class SV>
__global__ void __launch_bounds__(256) add_rows_kernel(SX* __restrict__ x, int64_t ld_x, const SA* __restrict__ a,
                                                       int64_t ld_a, const SV* __restrict__ vec, int64_t width) {
  const int64_t t = blockIdx.y;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < width; i += (int64_t)gridDim.x * blockDim.x) {
    float v = to_f32(x[t * ld_x + i]);
    if (a) v += to_f32(a[t * ld_a + i]);      // in this order: the rows first, then the vector
    if (vec) v += to_f32(vec[i]);
    x[t * ld_x + i] = from_f32<SX>(v);
  }
}

}  // namespace

// out[t, i] = alpha a[t, i] + beta b[t, i] (float arithmetic, one rounding); out may be a or b.
extern "C" int dinfer_axpby(int dtype, const void* a, int64_t ld_a, float alpha, const void* b, int64_t ld_b, float beta,
                            void* out, int64_t ld_out, int64_t rows, int64_t cols, hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return OK;
  if (rows > 65535) return ERR_BAD_SHAPE;
  const dim3 grid((unsigned)((cols + 255) / 256 < 64 ? (cols + 255) / 256 : 64), (unsigned)rows);
  DINFER_DISPATCH_DTYPE(dtype, {
    axpby_kernel<S><<<grid, 256, 0, stream>>>((const S*)a, ld_a, alpha, (const S*)b, ld_b, beta, (S*)out, ld_out, cols);
  });
  return launch_status();
}

// x[t, i] += a[t, i] + vec[i] (a and vec may each be null); x, a and vec each float or bf16.
extern "C" int dinfer_add_rows(void* x, int x_dtype, int64_t ld_x, const void* a, int a_dtype, int64_t ld_a,
                               const void* vec, int vec_dtype, int64_t rows, int64_t width, hipStream_t stream) {
  if (rows <= 0 || width <= 0) return OK;
  if (rows > 65535) return ERR_BAD_SHAPE;
  const dim3 grid((unsigned)((width + 255) / 256 < 64 ? (width + 255) / 256 : 64), (unsigned)rows);
#define ADD_ROWS(SX, SA, SV)                                                                                     \
  add_rows_kernel<SX, SA, SV><<<grid, 256, 0, stream>>>((SX*)x, ld_x, (const SA*)a, ld_a, (const SV*)vec, width)
  const int key = (x_dtype == DT_F32 ? 4 : 0) | (a_dtype == DT_F32 ? 2 : 0) | (vec_dtype == DT_F32 ? 1 : 0);
  for (int dt : {x_dtype, a_dtype, vec_dtype})
    if (dt != DT_F32 && dt != DT_BF16) return ERR_BAD_DTYPE;
  switch (key) {
    case 0: ADD_ROWS(bf16, bf16, bf16); break;
    case 1: ADD_ROWS(bf16, bf16, float); break;
    case 2: ADD_ROWS(bf16, float, bf16); break;
    case 3: ADD_ROWS(bf16, float, float); break;
    case 4: ADD_ROWS(float, bf16, bf16); break;
    case 5: ADD_ROWS(float, bf16, float); break;
    case 6: ADD_ROWS(float, float, bf16); break;
    default: ADD_ROWS(float, float, float); break;
  }
#undef ADD_ROWS
  return launch_status();
}
