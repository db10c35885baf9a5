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
enum { NORM_RMS = 0, NORM_LAYER = 1 };

struct StreamCoeffs {
  float in[STREAMS_MAX];
  float out[STREAMS_MAX];
  float mix[STREAMS_MAX * STREAMS_MAX];
};

// V values a thread and turn: 4 where rows and pointers allow 16-byte accesses (8-byte ones of bfloat16), else 1.
template <typename T, int V>
struct RowPiece {
  float v[V];
};
template <int V>
__device__ __forceinline__ RowPiece<float, V> load_piece(const float* p) {
  RowPiece<float, V> r;
  if constexpr (V == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    r.v[0] = t.x, r.v[1] = t.y, r.v[2] = t.z, r.v[3] = t.w;
  } else {
    r.v[0] = *p;
  }
  return r;
}
template <int V>
__device__ __forceinline__ RowPiece<float, V> load_piece(const bf16_t* p) {
  RowPiece<float, V> r;
  if constexpr (V == 4) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    r.v[0] = __uint_as_float(t.x << 16), r.v[1] = __uint_as_float(t.x & 0xffff0000u);
    r.v[2] = __uint_as_float(t.y << 16), r.v[3] = __uint_as_float(t.y & 0xffff0000u);
  } else {
    r.v[0] = bf16_bits_to_f32(*p);
  }
  return r;
}
template <int V>
__device__ __forceinline__ void store_piece(float* p, const float* v) {
  if constexpr (V == 4) *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  else *p = v[0];
}
template <int V>
__device__ __forceinline__ void store_piece(bf16_t* p, const float* v) {
  if constexpr (V == 4) *reinterpret_cast<uint2*>(p) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
  else *p = f32_to_bf16_bits(v[0]);
}

// One block per token, as many threads as the row has pieces (up to 1024): with rows of up to 4096 values every
// thread has all its loads on the way at once.
template <typename TY, typename TO, int V>
__global__ void __launch_bounds__(1024)
streams_step_kernel(float* __restrict__ streams, const TY* __restrict__ ya, const TY* __restrict__ yb, float a, float b,
                    const float* __restrict__ mix, const float* __restrict__ out_w, float mult,
                    const float* __restrict__ in_w, const float* __restrict__ gain, float eps, int kind,
                    TO* __restrict__ normed, const int* __restrict__ rows, int T, int H, int S, int write_back) {
  extern __shared__ __attribute__((aligned(16))) float u_row[];      // [H]: the mix the next sublayer reads
  __shared__ float scratch[16];
  __shared__ StreamCoeffs c;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int t = rows ? rows[blockIdx.x] : blockIdx.x;
  if (tid < S) {
    c.in[tid] = in_w ? in_w[tid] : 0.f;
    c.out[tid] = out_w ? out_w[tid] : 0.f;
  }
  if (mix != nullptr)
    for (int e = tid; e < S * S; e += nthreads) c.mix[e] = mix[e];
  __syncthreads();
  const bool has_branch = ya != nullptr;
  float sum = 0.f;
  for (int col = V * tid; col < H; col += V * nthreads) {
    RowPiece<float, V> x[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s)
      if (s < S) x[s] = load_piece<V>(streams + ((size_t)s * T + t) * H + col);
    if (has_branch) {
      RowPiece<float, V> y = load_piece<V>(ya + (size_t)t * H + col);
      if (yb != nullptr) {
        const RowPiece<float, V> y2 = load_piece<V>(yb + (size_t)t * H + col);
#pragma unroll
        for (int j = 0; j < V; ++j) y.v[j] = a * y.v[j] + b * y2.v[j];
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) y.v[j] = a * y.v[j];
      }
      RowPiece<float, V> nx[STREAMS_MAX];
#pragma unroll
      for (int to = 0; to < STREAMS_MAX; ++to) {
        if (to < S) {
#pragma unroll
          for (int j = 0; j < V; ++j) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < STREAMS_MAX; ++s)
              if (s < S) v += c.mix[s * S + to] * x[s].v[j];
            nx[to].v[j] = v + c.out[to] * (mult * y.v[j]);
          }
        }
      }
#pragma unroll
      for (int s = 0; s < STREAMS_MAX; ++s) {
        if (s < S) {
          x[s] = nx[s];
          if (write_back) store_piece<V>(streams + ((size_t)s * T + t) * H + col, nx[s].v);
        }
      }
    }
    if (gain != nullptr) {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s)
          if (s < S) u += c.in[s] * x[s].v[j];
        u_row[col + j] = u;
        sum += kind == NORM_LAYER ? u : u * u;
      }
    }
  }
  if (gain == nullptr) return;
  TO* dst = normed + (size_t)blockIdx.x * H;
  float mean = 0.f, r;
  if (kind == NORM_LAYER) {
    mean = block_sum(sum, scratch) / (float)H;
    float dev = 0.f;
    for (int col = V * tid; col < H; col += V * nthreads) {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float d = u_row[col + j] - mean;
        dev += d * d;
      }
    }
    r = 1.f / sqrtf(block_sum(dev, scratch) / (float)H + eps);
  } else {
    r = 1.f / sqrtf(block_sum(sum, scratch) / (float)H + eps);
  }
  for (int col = V * tid; col < H; col += V * nthreads) {
    float o[V];
#pragma unroll
    for (int j = 0; j < V; ++j) o[j] = (u_row[col + j] - mean) * r * gain[col + j];
    store_piece<V>(dst + col, o);
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
  const bool vec = H % 4 == 0 && ((uintptr_t)streams % 16) == 0 && ((uintptr_t)ya % 16) == 0 && ((uintptr_t)yb % 16) == 0 &&
                   ((uintptr_t)normed % 16) == 0;
  const int pieces = vec ? H / 4 : H;
  // few tokens: a thread per piece, so that every load of a row is on its way at once; many tokens: four pieces a
  // thread, smaller blocks and more of them resident (2048 tokens of 2048 values in two copies: 28.5 -> 21.5 us)
  const int per_thread = n >= 256 ? 4 : 1;
  int threads = 64;
  while (threads * per_thread < pieces && threads < 1024) threads *= 2;
#define STREAMS_GO_V(TY, TO, V)                                                                                      \
  do {                                                                                                               \
    if (shared > 48 * 1024) {                                                                                        \
      const hipError_t e = hipFuncSetAttribute((const void*)streams_step_kernel<TY, TO, V>,                          \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shared);             \
      if (e != hipSuccess) return (int)e;                                                                            \
    }                                                                                                                \
    hipLaunchKernelGGL((streams_step_kernel<TY, TO, V>), dim3(n), dim3(threads), shared, stream, streams,            \
                       (const TY*)ya, (const TY*)yb, a, b, mix, out_w, mult, in_w, gain, eps, kind, (TO*)normed,     \
                       rows, T_, H, S, write_back);                                                                  \
  } while (0)
#define STREAMS_GO(TY, TO) do { if (vec) STREAMS_GO_V(TY, TO, 4); else STREAMS_GO_V(TY, TO, 1); } while (0)
  if (y_dtype == ULLM_F32 && out_dtype == ULLM_F32) STREAMS_GO(float, float);
  else if (y_dtype == ULLM_F32 && out_dtype == ULLM_BF16) STREAMS_GO(float, bf16_t);
  else if (y_dtype == ULLM_BF16 && out_dtype == ULLM_F32) STREAMS_GO(bf16_t, float);
  else if (y_dtype == ULLM_BF16 && out_dtype == ULLM_BF16) STREAMS_GO(bf16_t, bf16_t);
  else return ULLM_ERR_DTYPE;
#undef STREAMS_GO
#undef STREAMS_GO_V
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
