// Several residual streams a token, mixed by learned weights around every sublayer ("hyper-connections").
//
// A token's row holds n streams of `width` floats side by side. Around a sublayer with input weights r[n], mixing
// matrix m[n, n] (indexed [from, to]) and output weights o[n]:
//
//   u = sum_s r[s] x_s          the sublayer's input (before its norm)
//   x_t <- sum_s m[s, t] x_s + o[t] y      all streams at once from the old ones, y the sublayer's output
//
//   streams_expand   every stream of a token starts as the same row (the embedding)
//   streams_step     one workgroup a token (the number of streams a template parameter, 16-byte moves) does what lies between two sublayers in one pass over the row: the write of
//                    the sublayer that has just run (optional), the read for the one that runs next (optional), and
//                    that one's layer norm with gain and bias (optional; without it u is written as float). With a list
//                    of source rows (the rows whose logits are wanted) nothing is stored into the streams.
//
// All arithmetic is float; the streams are float whatever the activations' type.
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int MAX_STREAMS = 8;

template <class S>
__global__ void __launch_bounds__(256) streams_expand_kernel(const S* __restrict__ src, int64_t ld_src,
                                                             float* __restrict__ x, int64_t ldx, int n, int width) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = to_f32(src[t * ld_src + c]);
    for (int s = 0; s < n; ++s) x[t * ldx + (int64_t)s * width + c] = v;
  }
}

struct Step {
  float* x; int64_t ldx; int n, width;
  const int32_t* rows;                       // source rows, or null: row = blockIdx.x and the streams are updated in place
  const void* branch; int64_t ld_branch;     // y, in the activations' type; null: no write
  const float* mix; const float* outw;       // [n, n], [n]
  const float* read;                         // [n], or null: no read
  const float* gain; const float* bias; float eps;   // layer norm of u; gain null: u itself goes to `u_out`
  void* out; int64_t ld_out;                 // normed u in the activations' type
  float* u_out; int64_t ld_u;
};

// N streams (a template parameter: every array below stays in registers), VEC consecutive columns a thread and pass.
template <class S, int N, int VEC>
__global__ void __launch_bounds__(256) streams_step_kernel(Step p) {
  extern __shared__ float us[];              // u of this row
  __shared__ float red[16];
  const int W = p.width;
  float mix[N][N], outw[N], readw[N];
#pragma unroll
  for (int s = 0; s < N; ++s) {
    outw[s] = p.branch ? p.outw[s] : 0.f;
    readw[s] = p.read ? p.read[s] : 0.f;
#pragma unroll
    for (int to = 0; to < N; ++to) mix[s][to] = p.branch ? p.mix[s * N + to] : 0.f;
  }
  const int64_t r = blockIdx.x;
  const int64_t t = p.rows ? p.rows[r] : r;
  float* xr = p.x + t * p.ldx;
  const S* y = p.branch ? (const S*)p.branch + t * p.ld_branch : nullptr;
  float sum = 0.f;
  for (int c = threadIdx.x * VEC; c < W; c += 256 * VEC) {
    float xs[N][VEC];
#pragma unroll
    for (int s = 0; s < N; ++s) {
      if (VEC == 4) {
        const f32x4 v = *(const f32x4*)(xr + (int64_t)s * W + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) xs[s][e] = v[e];
      } else {
        xs[s][0] = xr[(int64_t)s * W + c];
      }
    }
    if (y) {
      float yv[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) yv[e] = to_f32(y[c + e]);
      float nx[N][VEC];
#pragma unroll
      for (int to = 0; to < N; ++to)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < N; ++s) acc = __builtin_fmaf(mix[s][to], xs[s][e], acc);
          nx[to][e] = __builtin_fmaf(outw[to], yv[e], acc);
        }
#pragma unroll
      for (int s = 0; s < N; ++s) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) xs[s][e] = nx[s][e];
        if (!p.rows) {
          if (VEC == 4) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = nx[s][e];
            *(f32x4*)(xr + (int64_t)s * W + c) = v;
          } else {
            xr[(int64_t)s * W + c] = nx[s][0];
          }
        }
      }
    }
    if (p.read) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < N; ++s) u = __builtin_fmaf(readw[s], xs[s][e], u);
        if (p.gain) {
          us[c + e] = u;
          sum += u;
        } else {
          p.u_out[r * p.ld_u + c + e] = u;
        }
      }
    }
  }
  if (!p.read || !p.gain) return;
  const float mean = block_sum(sum, red) / (float)W;
  float sq = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float d = us[c] - mean;
    sq = __builtin_fmaf(d, d, sq);
  }
  const float inv = 1.f / sqrtf(block_sum(sq, red) / (float)W + p.eps);
  S* o = (S*)p.out + r * p.ld_out;
  for (int c = threadIdx.x; c < W; c += 256)
    o[c] = from_f32<S>((us[c] - mean) * inv * p.gain[c] + (p.bias ? p.bias[c] : 0.f));
}

template <class S, int VEC>
void launch_step(const Step& p, int64_t n_rows, size_t lds, hipStream_t stream) {
  const unsigned g = (unsigned)n_rows;
  switch (p.n) {
    case 1: streams_step_kernel<S, 1, VEC><<<g, 256, lds, stream>>>(p); break;
    case 2: streams_step_kernel<S, 2, VEC><<<g, 256, lds, stream>>>(p); break;
    case 3: streams_step_kernel<S, 3, VEC><<<g, 256, lds, stream>>>(p); break;
    case 4: streams_step_kernel<S, 4, VEC><<<g, 256, lds, stream>>>(p); break;
    case 5: streams_step_kernel<S, 5, VEC><<<g, 256, lds, stream>>>(p); break;
    case 6: streams_step_kernel<S, 6, VEC><<<g, 256, lds, stream>>>(p); break;
    case 7: streams_step_kernel<S, 7, VEC><<<g, 256, lds, stream>>>(p); break;
    default: streams_step_kernel<S, 8, VEC><<<g, 256, lds, stream>>>(p); break;
  }
}

}  // namespace

// x[t, s width + c] = src[t, c] for every stream s < n; src in the type `dtype`, x float.
extern "C" int dinfer_streams_expand(int dtype, const void* src, int64_t ld_src, float* x, int64_t ldx, int64_t tokens,
                                     int n, int width, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (n <= 0 || width <= 0 || ldx < (int64_t)n * width || tokens > 0x7fffffff) return ERR_BAD_SHAPE;
  DINFER_DISPATCH_DTYPE(dtype, {
    streams_expand_kernel<S><<<(unsigned)tokens, 256, 0, stream>>>((const S*)src, ld_src, x, ldx, n, width);
  });
  return launch_status();
}

// See the head of the file. dtype: the type of branch and out. rows: int32 source rows of the n_rows rows worked on
// (then the streams stay as they are), or null for rows 0 .. n_rows - 1.
extern "C" int dinfer_streams_step(int dtype, float* x, int64_t ldx, int n, int width, const int32_t* rows,
                                   const void* branch, int64_t ld_branch, const float* mix, const float* outw,
                                   const float* read, const float* gain, const float* bias, float eps, void* out,
                                   int64_t ld_out, float* u_out, int64_t ld_u, int64_t n_rows, hipStream_t stream) {
  if (n_rows <= 0) return OK;
  if (n <= 0 || width <= 0 || ldx < (int64_t)n * width || n_rows > 0x7fffffff) return ERR_BAD_SHAPE;
  if (n > MAX_STREAMS || width > 12288) return ERR_UNSUPPORTED;   // a row of u waits in LDS
  if (branch && (!mix || !outw)) return ERR_BAD_SHAPE;
  if (read && (gain ? !out : !u_out)) return ERR_BAD_SHAPE;
  if (!branch && !read) return OK;
  Step p{x, ldx, n, width, rows, branch, ld_branch, mix, outw, read, gain, bias, eps, out, ld_out, u_out, ld_u};
  const size_t lds = (read && gain) ? (size_t)width * sizeof(float) : 0;
  // 16-byte moves where every stream of every row starts on a 16-byte boundary
  const bool vec = width % 4 == 0 && ldx % 4 == 0 && ((uintptr_t)x % 16) == 0;
  DINFER_DISPATCH_DTYPE(dtype, {
    if (vec) launch_step<S, 4>(p, n_rows, lds, stream);
    else launch_step<S, 1>(p, n_rows, lds, stream);
  });
  return launch_status();
}
