// A residual stream kept in several copies (hyper-connections).  The copies are float32 [S, T, H].  A sublayer
// reads one mix of them, u = sum_s in[s] x_s, and writes back into all of them at once from the old ones:
// x_t <- sum_s mix[s, t] x_s + mult * out[t] * y   (mix is indexed [from, to]).
//
// One kernel does what lies between two sublayers: the write-back of the sublayer before (if there is a branch y,
// which may be the weighted sum ya * a + yb * b of two branches) and the read and norm for the sublayer after (if
// there is a gain).  With `rows` only the listed tokens are worked on and nothing is written back (the last norm
// of a model, for the rows whose logits are wanted).  Everything is 32-bit; a row's sums have a fixed order.
#include "common.h"

#define STREAMS_MAX 8
#define STREAMS_THREADS 256
enum { NORM_RMS = 0, NORM_LAYER = 1 };

struct StreamCoeffs {
  float in[STREAMS_MAX];
  float out[STREAMS_MAX];
  float mix[STREAMS_MAX * STREAMS_MAX];
};

template <typename TY, typename TO>
__global__ void __launch_bounds__(STREAMS_THREADS)
streams_step_kernel(float* __restrict__ streams, const TY* __restrict__ ya, const TY* __restrict__ yb, float a, float b,
                    const float* __restrict__ mix, const float* __restrict__ out_w, float mult,
                    const float* __restrict__ in_w, const float* __restrict__ gain, float eps, int kind,
                    TO* __restrict__ normed, const int* __restrict__ rows, int T, int H, int S, int write_back) {
  extern __shared__ float u_row[];                  // [H]: the mix the next sublayer reads
  __shared__ float scratch[16];
  __shared__ StreamCoeffs c;
  const int tid = threadIdx.x;
  const int t = rows ? rows[blockIdx.x] : blockIdx.x;
  if (tid < S) {
    c.in[tid] = in_w ? in_w[tid] : 0.f;
    c.out[tid] = out_w ? out_w[tid] : 0.f;
  }
  if (mix != nullptr)
    for (int e = tid; e < S * S; e += STREAMS_THREADS) c.mix[e] = mix[e];
  __syncthreads();
  const bool has_branch = ya != nullptr;
  float sum = 0.f;
  for (int col = tid; col < H; col += STREAMS_THREADS) {
    float x[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < S) x[s] = streams[((size_t)s * T + t) * H + col];
    if (has_branch) {
      float y = a * ld_f32(ya + (size_t)t * H + col);
      if (yb != nullptr) y += b * ld_f32(yb + (size_t)t * H + col);
      y *= mult;
      float nx[STREAMS_MAX];
#pragma unroll
      for (int to = 0; to < STREAMS_MAX; ++to) {
        if (to < S) {
          float v = 0.f;
#pragma unroll
          for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < S) v += c.mix[s * S + to] * x[s];
          nx[to] = v + c.out[to] * y;
        }
      }
#pragma unroll
      for (int s = 0; s < STREAMS_MAX; ++s) {
        if (s < S) {
          x[s] = nx[s];
          if (write_back) streams[((size_t)s * T + t) * H + col] = nx[s];
        }
      }
    }
    if (gain != nullptr) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < STREAMS_MAX; ++s)
        if (s < S) u += c.in[s] * x[s];
      u_row[col] = u;
      sum += kind == NORM_LAYER ? u : u * u;
    }
  }
  if (gain == nullptr) return;
  TO* dst = normed + (size_t)blockIdx.x * H;
  if (kind == NORM_LAYER) {
    const float mean = block_sum(sum, scratch) / (float)H;
    float dev = 0.f;
    for (int col = tid; col < H; col += STREAMS_THREADS) {
      const float d = u_row[col] - mean;
      dev += d * d;
    }
    const float r = 1.f / sqrtf(block_sum(dev, scratch) / (float)H + eps);
    for (int col = tid; col < H; col += STREAMS_THREADS) st_f32(dst + col, (u_row[col] - mean) * r * gain[col]);
  } else {
    const float r = 1.f / sqrtf(block_sum(sum, scratch) / (float)H + eps);
    for (int col = tid; col < H; col += STREAMS_THREADS) st_f32(dst + col, u_row[col] * r * gain[col]);
  }
}

// streams [S, T, H] float32.  ya / yb: branches [T, H] of dtype y_dtype (yb and ya may be null); normed [n, H] of
// out_dtype (null with gain null).  rows: int32 [n] or null (then n == T and the streams are written back).
extern "C" int ullm_streams_step(float* streams, const void* ya, const void* yb, float a, float b, int y_dtype,
                                 const float* mix, const float* out_w, float mult, const float* in_w, const float* gain,
                                 float eps, int kind, void* normed, int out_dtype, const int* rows, int n, int T_, int H,
                                 int S, hipStream_t stream) {
  if (n <= 0) return 0;
  if (S < 1 || S > STREAMS_MAX || H < 1 || T_ < 1) return ULLM_ERR_SHAPE;
  if (ya == nullptr && yb != nullptr) return ULLM_ERR_UNSUPPORTED;
  if (ya != nullptr && (mix == nullptr || out_w == nullptr)) return ULLM_ERR_UNSUPPORTED;
  if (gain != nullptr && (in_w == nullptr || normed == nullptr)) return ULLM_ERR_UNSUPPORTED;
  if (kind != NORM_RMS && kind != NORM_LAYER) return ULLM_ERR_UNSUPPORTED;
  const size_t shared = gain ? (size_t)H * sizeof(float) : 0;
  if (shared > 160 * 1024 - 4096) return ULLM_ERR_SHAPE;
  const int write_back = rows == nullptr ? 1 : 0;
#define STREAMS_GO(TY, TO)                                                                                           \
  do {                                                                                                               \
    if (shared > 48 * 1024) {                                                                                        \
      const hipError_t e = hipFuncSetAttribute((const void*)streams_step_kernel<TY, TO>,                             \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shared);             \
      if (e != hipSuccess) return (int)e;                                                                            \
    }                                                                                                                \
    hipLaunchKernelGGL((streams_step_kernel<TY, TO>), dim3(n), dim3(STREAMS_THREADS), shared, stream, streams,       \
                       (const TY*)ya, (const TY*)yb, a, b, mix, out_w, mult, in_w, gain, eps, kind, (TO*)normed,     \
                       rows, T_, H, S, write_back);                                                                  \
  } while (0)
  if (y_dtype == ULLM_F32 && out_dtype == ULLM_F32) STREAMS_GO(float, float);
  else if (y_dtype == ULLM_F32 && out_dtype == ULLM_BF16) STREAMS_GO(float, bf16_t);
  else if (y_dtype == ULLM_BF16 && out_dtype == ULLM_F32) STREAMS_GO(bf16_t, float);
  else if (y_dtype == ULLM_BF16 && out_dtype == ULLM_BF16) STREAMS_GO(bf16_t, bf16_t);
  else return ULLM_ERR_DTYPE;
#undef STREAMS_GO
  ULLM_LAUNCH_CHECK();
}

// out[s, t, :] = x[t, :] for every s: the copies of the stream all start as the embedding output.
__global__ void __launch_bounds__(256)
streams_spread_kernel(const float* __restrict__ x, float* __restrict__ out, size_t n, int S) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = x[i];
  for (int s = 0; s < S; ++s) out[(size_t)s * n + i] = v;
}

extern "C" int ullm_streams_spread(const float* x, float* out, long long n, int S, hipStream_t stream) {
  if (n <= 0) return 0;
  if (S < 1) return ULLM_ERR_SHAPE;
  hipLaunchKernelGGL(streams_spread_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, out, (size_t)n, S);
  ULLM_LAUNCH_CHECK();
}

// out = a * x + b * y in 32-bit: the sum of two mixers that run side by side, each with a weight.
template <typename TX, typename TY>
__global__ void __launch_bounds__(256)
weighted_sum_kernel(const TX* __restrict__ x, const TY* __restrict__ y, float a, float b, float* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = a * ld_f32(x + i) + b * ld_f32(y + i);
}

extern "C" int ullm_weighted_sum(const void* x, int x_dtype, const void* y, int y_dtype, float a, float b, float* out,
                                 long long n, hipStream_t stream) {
  if (n <= 0) return 0;
  const dim3 grid((unsigned)((n + 255) / 256));
#define WS_GO(TX, TY) hipLaunchKernelGGL((weighted_sum_kernel<TX, TY>), grid, dim3(256), 0, stream, (const TX*)x, (const TY*)y, a, b, out, (size_t)n)
  if (x_dtype == ULLM_F32 && y_dtype == ULLM_F32) WS_GO(float, float);
  else if (x_dtype == ULLM_F32 && y_dtype == ULLM_BF16) WS_GO(float, bf16_t);
  else if (x_dtype == ULLM_BF16 && y_dtype == ULLM_F32) WS_GO(bf16_t, float);
  else if (x_dtype == ULLM_BF16 && y_dtype == ULLM_BF16) WS_GO(bf16_t, bf16_t);
  else return ULLM_ERR_DTYPE;
#undef WS_GO
  ULLM_LAUNCH_CHECK();
}
