// Latent attention: queries, keys and values that go through small latents.
//
// Per token the mixer's first product leaves one 32-bit row  [ q latent | kv latent | rotated key part | head gates ].
// The cache holds, per token, ONE key row for all heads, [ c | k_rot | 0.. ] with c = rmsnorm(kv latent) * gain
// and k_rot the rotated key part turned by the token's position, and the same c as the value row (transposed
// inside the page, as the attention kernels read values).  With q'_h = W_uk[h]^T q_plain[h] the score of head h is
//     q_plain[h] . (W_uk[h] c) + q_rot[h] . k_rot  =  [ q'_h | q_rot[h] ] . [ c | k_rot ],
// so attention runs as grouped-query attention with one key/value head of size kv_rank + rot_dim over the
// latent cache, and a head's output  sum_j p_j c_j  is taken through W_uv[h] afterwards.
//
//   latent_prepare   the two norms, the key part's rotation, the cache write, the gate logits in the compute dtype
//   head_linear      y[t, h, :] = W[h]^T x[t, h, :] for a matrix per head (q' from q_plain; values from latent outputs)
//   latent_query     [ q'_h | rotate(q_rot[h]) | 0.. ] per head, the query rows the attention kernels take
//
// All arithmetic is 32-bit; T selects the storage type only.  Sums run in an order that depends on the row alone.
#include "common.h"

// ------------------------------------------------------------------ norms, rotation, cache write
// One block per token.  proj float32 [T, ld]: q latent at q_off (q_rank values), kv latent at kv_off (kv_rank), the
// rotated key part at kr_off (rot, half-split pairs (i, i + rot/2), cos/sin = table[pos, i], table[pos, rot/2 + i]),
// gate logits at g_off (n_gate values; n_gate 0: none).
// Outputs: cq [T, q_rank] = rmsnorm(q latent) * q_gain; key pool row [page, 0, slot, 0 .. kv_rank + rot) and value
// pool column [page, 0, 0 .. kv_rank, slot] (pools made for one head of size hd >= kv_rank + rot; the dims behind
// are never written and stay zero); gate [T, ldg] = the gate logits and zeros behind them.  Tokens whose page id is negative write no cache.
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const float* __restrict__ proj, int ld, int q_off, int q_rank, int kv_off, int kv_rank, int kr_off,
                      int rot, int g_off, int n_gate, const float* __restrict__ q_gain, const float* __restrict__ kv_gain,
                      float eps, const float* __restrict__ cos_sin, int table_rows, const int* __restrict__ positions,
                      const int* __restrict__ token_entry, const int* __restrict__ block_table, int bt_stride,
                      T* __restrict__ k_pool, T* __restrict__ v_pool, int page_size, int hd, int write_kv,
                      T* __restrict__ cq, T* __restrict__ gate, int ldg) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* row = proj + (size_t)t * ld;
  const int pos = positions[t];
  if (q_rank > 0) {
    float ss = 0.f;
    for (int i = tid; i < q_rank; i += 256) ss = fmaf(row[q_off + i], row[q_off + i], ss);
    ss = block_sum(ss, scratch);
    const float rs = rsqrtf(ss / (float)q_rank + eps);
    for (int i = tid; i < q_rank; i += 256) st_f32(cq + (size_t)t * q_rank + i, (row[q_off + i] * rs) * q_gain[i]);
  }
  for (int i = tid; i < (n_gate ? ldg : 0); i += 256) st_f32(gate + (size_t)t * ldg + i, i < n_gate ? row[g_off + i] : 0.f);
  if (!write_kv) return;
  const int page = block_table[(size_t)token_entry[t] * bt_stride + pos / page_size];
  float ss = 0.f;
  for (int i = tid; i < kv_rank; i += 256) ss = fmaf(row[kv_off + i], row[kv_off + i], ss);
  ss = block_sum(ss, scratch);
  if (page < 0) return;
  const float rs = rsqrtf(ss / (float)kv_rank + eps);
  const int slot = pos % page_size;
  T* kdst = k_pool + ((size_t)page * page_size + slot) * hd;
  T* vdst = v_pool + (size_t)page * hd * page_size + slot;
  for (int i = tid; i < kv_rank; i += 256) {
    const float c = (row[kv_off + i] * rs) * kv_gain[i];
    st_f32(kdst + i, c);
    st_f32(vdst + (size_t)i * page_size, c);
  }
  const int half = rot / 2;
  const int p = pos < table_rows ? pos : table_rows - 1;    // the host rejects positions past the table
  for (int i = tid; i < half; i += 256) {
    const float c = cos_sin[(size_t)p * rot + i], s = cos_sin[(size_t)p * rot + half + i];
    const float a = row[kr_off + i], b = row[kr_off + half + i];
    st_f32(kdst + kv_rank + i, a * c - b * s);
    st_f32(kdst + kv_rank + half + i, b * c + a * s);
  }
}

extern "C" int ullm_latent_prepare(const float* proj, int ld, int q_off, int q_rank, int kv_off, int kv_rank, int kr_off,
                                   int rot, int g_off, int n_gate, const float* q_gain, const float* kv_gain, float eps,
                                   const float* cos_sin, int table_rows, const int* positions, const int* token_entry,
                                   const int* block_table, int bt_stride, void* k_pool, void* v_pool, int page_size,
                                   int hd, int write_kv, void* cq, void* gate, int ldg, int T_, int dtype,
                                   hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (q_rank < 0 || kv_rank < 1 || rot < 0 || (rot & 1) || n_gate < 0 || hd < kv_rank + rot || page_size < 1)
    return ULLM_ERR_SHAPE;
  if (q_off < 0 || q_off + q_rank > ld || kv_off < 0 || kv_off + kv_rank > ld || kr_off < 0 || kr_off + rot > ld ||
      g_off < 0 || g_off + n_gate > ld || (n_gate > 0 && ldg < n_gate))
    return ULLM_ERR_SHAPE;
  if (rot > 0 && (!cos_sin || table_rows <= 0)) return ULLM_ERR_SHAPE;
#define GO(TT) hipLaunchKernelGGL(latent_prepare_kernel<TT>, dim3(T_), dim3(256), 0, stream, proj, ld, q_off, q_rank, kv_off, \
    kv_rank, kr_off, rot, g_off, n_gate, q_gain, kv_gain, eps, cos_sin, table_rows, positions, token_entry, block_table,       \
    bt_stride, (TT*)k_pool, (TT*)v_pool, page_size, hd, write_kv, (TT*)cq, (TT*)gate, ldg)
  if (dtype == ULLM_F32) GO(float);
  else if (dtype == ULLM_BF16) GO(bf16_t);
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ a matrix per head
// y[t, h, n] = sum_k x[t, h, k] * w[h, k, n]:  x [T, heads, K] with strides (x_st, x_sh, 1), w contiguous
// [heads, K, N] (a row of w holds one input's weights for all outputs, so a wave's loads of a row are one
// contiguous piece), y [T, heads, N] with strides (y_st, y_sh, 1).  grid (token tiles of HL_TOKENS, heads, chunks
// of 64 * NV outputs); the tile's rows of x lie in shared memory as 32-bit values; a lane owns NV adjacent
// outputs, wave j of the HL_WAVES takes k = j, j + HL_WAVES, ... in rising order (eight rows of w under way at a
// time: few rows are bound by the loads' latency, not their bytes), and the waves' partial sums are added in wave
// order through shared memory: an order that depends on the row alone.  A fetched row of w serves all the tile's
// tokens.
#define HL_TOKENS 8
#define HL_WAVES 8
#define HL_THREADS (64 * HL_WAVES)
template <typename T, int NV>
__device__ __forceinline__ void hl_load(const T* p, bool ok, float (&v)[NV]) {
  if constexpr (NV == 1) {
    v[0] = ok ? ld_f32(p) : 0.f;
  } else if constexpr (sizeof(T) == 2) {
    const uint32_t u = ok ? *reinterpret_cast<const uint32_t*>(p) : 0u;
    v[0] = __builtin_bit_cast(float, u << 16);
    v[1] = __builtin_bit_cast(float, u & 0xffff0000u);
  } else {
    const float2 f = ok ? *reinterpret_cast<const float2*>(p) : make_float2(0.f, 0.f);
    v[0] = f.x;
    v[1] = f.y;
  }
}

template <typename T, int NV>
__global__ void __launch_bounds__(HL_THREADS)
head_linear_kernel(const T* __restrict__ x, long long x_st, long long x_sh, const T* __restrict__ w,
                   T* __restrict__ y, long long y_st, long long y_sh, int n_tokens, int N, int K) {
  extern __shared__ float hl_shared[];
  float* xs = hl_shared;                                               // [HL_TOKENS][K]
  float* part = hl_shared + (size_t)HL_TOKENS * K;                     // [HL_WAVES][HL_TOKENS][64 * NV]
  constexpr int CH = 64 * NV, W = HL_WAVES, U = 8;
  const int t0 = blockIdx.x * HL_TOKENS, h = blockIdx.y, n0 = blockIdx.z * CH;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_rows = n_tokens - t0 < HL_TOKENS ? n_tokens - t0 : HL_TOKENS;
  for (int i = tid; i < HL_TOKENS * K; i += HL_THREADS) {
    const int r = i / K, k = i - r * K;
    xs[i] = r < n_rows ? ld_f32(x + (size_t)(t0 + r) * x_st + (size_t)h * x_sh + k) : 0.f;
  }
  __syncthreads();
  const int n = n0 + lane * NV;
  const bool ok = n < N;                                               // NV == 2 only where N is even: both or none
  const T* wp = w + (size_t)h * K * N + n;
  float acc[HL_TOKENS][NV];
#pragma unroll
  for (int r = 0; r < HL_TOKENS; ++r)
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[r][v] = 0.f;
  int k = wave;
  for (; k + (U - 1) * W < K; k += U * W) {                            // U rows of w under way
    float wv[U][NV];
#pragma unroll
    for (int u = 0; u < U; ++u) hl_load<T, NV>(wp + (size_t)(k + u * W) * N, ok, wv[u]);
#pragma unroll
    for (int r = 0; r < HL_TOKENS; ++r)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float xv = xs[r * K + k + u * W];
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[r][v] = fmaf(xv, wv[u][v], acc[r][v]);
      }
  }
  for (; k < K; k += W) {
    float w0[NV];
    hl_load<T, NV>(wp + (size_t)k * N, ok, w0);
#pragma unroll
    for (int r = 0; r < HL_TOKENS; ++r)
#pragma unroll
      for (int v = 0; v < NV; ++v) acc[r][v] = fmaf(xs[r * K + k], w0[v], acc[r][v]);
  }
#pragma unroll
  for (int r = 0; r < HL_TOKENS; ++r)
#pragma unroll
    for (int v = 0; v < NV; ++v) part[((size_t)wave * HL_TOKENS + r) * CH + lane * NV + v] = acc[r][v];
  __syncthreads();
  for (int o = tid; o < HL_TOKENS * CH; o += HL_THREADS) {
    const int r = o / CH, c = o - r * CH;
    if (r >= n_rows || n0 + c >= N) continue;
    float s = part[o];
#pragma unroll
    for (int j = 1; j < W; ++j) s += part[(size_t)j * HL_TOKENS * CH + o];
    st_f32(y + (size_t)(t0 + r) * y_st + (size_t)h * y_sh + n0 + c, s);
  }
}

extern "C" int ullm_head_linear(const void* x, long long x_st, long long x_sh, const void* w, void* y, long long y_st,
                                long long y_sh, int T_, int heads, int N, int K, int dtype, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (heads < 1 || heads > 65535 || N < 1 || K < 1 || K > 1024) return ULLM_ERR_SHAPE;      // the rows in shared memory
  if (dtype != ULLM_F32 && dtype != ULLM_BF16) return ULLM_ERR_DTYPE;
  // two outputs a lane where a pair is one aligned load and the outputs fill at least a wave that way
  const int nv = (N % 2 == 0 && N >= 128) ? 2 : 1;
  const int chunk = 64 * nv;
  if ((N + chunk - 1) / chunk > 65535) return ULLM_ERR_SHAPE;
  dim3 grid((T_ + HL_TOKENS - 1) / HL_TOKENS, heads, (N + chunk - 1) / chunk), block(HL_THREADS);
  const size_t lds = ((size_t)K * HL_TOKENS + (size_t)HL_WAVES * HL_TOKENS * chunk) * sizeof(float);
#define GO(TT, NV) hipLaunchKernelGGL((head_linear_kernel<TT, NV>), grid, block, lds, stream, (const TT*)x, x_st, x_sh, \
    (const TT*)w, (TT*)y, y_st, y_sh, T_, N, K)
  if (dtype == ULLM_F32) { if (nv == 2) GO(float, 2); else GO(float, 1); }
  else { if (nv == 2) GO(bf16_t, 2); else GO(bf16_t, 1); }
#undef GO
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ the query rows of the attention kernels
// out[t, h, :] = [ qa[t, h, 0 .. rank) | rotate(q[t, h, plain .. plain + rot)) | zeros up to hd ]:  qa with strides
// (qa_st, qa_sh, 1); q [T, heads * (plain + rot)] the up-projected queries, whose last rot dims per head are
// turned by the token's position (half-split pairs, table as above).  One block of LQ_THREADS per (token, head).
#define LQ_THREADS 128
template <typename T>
__global__ void __launch_bounds__(LQ_THREADS)
latent_query_kernel(const T* __restrict__ qa, long long qa_st, long long qa_sh, const T* __restrict__ q, int ldq,
                    int plain, int rot, int rank, int heads, int hd, const float* __restrict__ cos_sin, int table_rows,
                    const int* __restrict__ positions, T* __restrict__ out, int ldo) {
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[t], half = rot / 2;
  const int p = pos < table_rows ? pos : table_rows - 1;
  const float* cs = cos_sin + (size_t)p * rot;
  for (int d = tid; d < hd; d += LQ_THREADS) {
    float v = 0.f;
    if (d < rank) {
      v = ld_f32(qa + (size_t)t * qa_st + (size_t)h * qa_sh + d);
    } else if (d < rank + rot) {
      const int j = d - rank;
      const T* qr = q + (size_t)t * ldq + (size_t)h * (plain + rot) + plain;
      if (j < half) v = ld_f32(qr + j) * cs[j] - ld_f32(qr + j + half) * cs[half + j];
      else v = ld_f32(qr + j) * cs[j - half] + ld_f32(qr + j - half) * cs[j];
    }
    st_f32(out + (size_t)t * ldo + (size_t)h * hd + d, v);
  }
}

extern "C" int ullm_latent_query(const void* qa, long long qa_st, long long qa_sh, const void* q, int ldq, int plain,
                                 int rot, int rank, int heads, int hd, const float* cos_sin, int table_rows,
                                 const int* positions, void* out, int ldo, int T_, int dtype, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (heads < 1 || heads > 65535 || plain < 0 || rot < 0 || (rot & 1) || rank < 1 || hd < rank + rot ||
      ldq < heads * (plain + rot) || ldo < heads * hd)
    return ULLM_ERR_SHAPE;
  if (rot > 0 && (!cos_sin || table_rows <= 0)) return ULLM_ERR_SHAPE;
#define GO(TT) hipLaunchKernelGGL(latent_query_kernel<TT>, dim3(T_, heads), dim3(LQ_THREADS), 0, stream, (const TT*)qa, qa_st, qa_sh, \
    (const TT*)q, ldq, plain, rot, rank, heads, hd, cos_sin, table_rows, positions, (TT*)out, ldo)
  if (dtype == ULLM_F32) GO(float);
  else if (dtype == ULLM_BF16) GO(bf16_t);
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}
