// Routed feed-forward (mixture of experts): routing, the grouping of (token, chosen expert) pairs by expert,
// the experts' two products over the grouped rows, and the weighted sum.  Nothing here waits for the device
// or sizes a launch by values: grids are made for the most tiles any routing can give, and a block whose
// tile is empty leaves at once, so a step can be captured into a graph.
//
//   route     logits [T, R] (R = experts with weights + identity experts) -> softmax over all R, the choice by
//             softmax + correction, the `top` largest (ties: the lower index), weights = the chosen experts'
//             softmax values over their sum (+ 1e-20).  Or (mode ROUTE_TOP_LOGITS) the `top` largest of logits +
//             bias, weights = the softmax over those alone.  Or (mode ROUTE_SIGMOID) scores = sigmoid(logit) each on
//             its own, the choice by score + correction, weights = the chosen scores over their sum (+ 1e-20).  The
//             weights are multiplied by one constant.  All 32-bit.  One wave per token.
//   sort      pairs (token, k) -> rows ("slots") grouped by expert; identity experts (index >= experts) get no
//             slot.  Which slot inside its expert a pair gets depends on timing; no value does: every row of a
//             product is a function of that row alone.  Also the tile list: (expert, first slot, rows <= tile_rows).
//   gate_up   act[slot, :] = glu(x[token of slot] Wg[e]^T, x Wu[e]^T) with the clamped gated unit
//             g' = min(g, limit), u' = clamp(u, -limit, limit), act = g' sigmoid(alpha g') (u' + 1),
//             or without a limit (limit <= 0) the plain unit silu(g) u
//   down      y[slot, :] = act[slot] Wd[e]^T, 32-bit
//   combine   out[t] = base[t] + bias + shared[t] + sum_k weight[t, k] * (expert k has weights ? y[slot(t, k)] : x[t]),
//             added in the order of k, 32-bit.
//
// Products: bfloat16 on v_mfma_f32_16x16x32_bf16 (A operand = 16 rows of an expert's matrix, lane (r, g) holds
// W[n0 + r][k + 8g .. +8]; B operand = 16 grouped rows of x; lane (r, g) then holds out[row r][column n0 + 4g .. +4]),
// or for float32 and for shapes the tiles do not take a kernel with one wave per output value that sums K in a
// fixed order.  Expert matrices are stacked: gate|up [experts, 2 ff, hidden], down [experts, hidden, ff].
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
union Pack8 {
  bf16x8_t v;
  uint4 u4;
};

#define MOE_MAX_ROUTER 1024          // router outputs (experts + identity experts)
#define MOE_MAX_TOP 32

// ------------------------------------------------------------------------------- routing
// One wave: softmax over the logits z[0 .. n_router) in shared memory (overwritten by the scores), the `top` largest
// of score + correction, the chosen scores over their sum.  s_choice holds n_router floats, s_pick MOE_MAX_TOP.
// mode ROUTE_TOP_LOGITS: `correction` is a bias on the logits; the `top` largest of logit + bias are chosen and
// weighed by the softmax over the chosen ones alone.
// mode ROUTE_SIGMOID: every score is the sigmoid of its own logit; choice and weights as for ROUTE_SOFTMAX_ALL.
// Every weight is multiplied by `weight_scale`.
enum { ROUTE_SOFTMAX_ALL = 0, ROUTE_TOP_LOGITS = 1, ROUTE_SIGMOID = 2 };
__device__ __forceinline__ void route_from_logits(float* z, float* s_choice, float* s_pick,
                                                  const float* __restrict__ correction, int n_router, int top,
                                                  int* __restrict__ ids, float* __restrict__ weights, int lane,
                                                  int mode, float weight_scale) {
  if (mode == ROUTE_TOP_LOGITS) {
    for (int e = lane; e < n_router; e += 64) {
      const float v = z[e] + (correction ? correction[e] : 0.f);
      z[e] = v;
      s_choice[e] = v;
    }
  } else if (mode == ROUTE_SIGMOID) {
    for (int e = lane; e < n_router; e += 64) {
      const float s = 1.f / (1.f + expf(-z[e]));
      z[e] = s;
      s_choice[e] = s + (correction ? correction[e] : 0.f);
    }
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < n_router; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < n_router; e += 64) {
      const float p = expf(z[e] - mx);
      z[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < n_router; e += 64) {
      const float s = z[e] / sum;
      z[e] = s;
      s_choice[e] = s + (correction ? correction[e] : 0.f);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < n_router; e += 64) {
      const float c = s_choice[e];
      if (c > best || (c == best && e < at)) {
        best = c;
        at = e;
      }
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) {
      const float ob = __shfl_xor(best, m, 64);
      const int oa = __shfl_xor(at, m, 64);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at >= n_router) at = k < n_router ? k : 0;       // every value a NaN: any expert
    const float s = z[at];
    total += s;
    if (lane == 0) {
      ids[k] = at;
      s_pick[k] = s;
      s_choice[at] = -INFINITY;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
  }
  if (mode == ROUTE_TOP_LOGITS) {
    // the first pick is the largest: softmax over the picked logits, added in the order they were picked
    const float mx = s_pick[0];
    float sum = 0.f;
    for (int k = 0; k < top; ++k) sum += expf(s_pick[k] - mx);
    if (lane < top) weights[lane] = expf(s_pick[lane] - mx) / sum * weight_scale;
    return;
  }
  if (lane < top) weights[lane] = s_pick[lane] / (total + 1e-20f) * weight_scale;
}

__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ correction, int n_router, int top,
                 int* __restrict__ ids, float* __restrict__ weights, int mode, float weight_scale) {
  __shared__ float s_soft[MOE_MAX_ROUTER], s_choice[MOE_MAX_ROUTER];
  __shared__ float s_pick[MOE_MAX_TOP];
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < n_router; e += 64) s_soft[e] = logits[(size_t)t * ld + e];
  __syncthreads();
  route_from_logits(s_soft, s_choice, s_pick, correction, n_router, top, ids + (size_t)t * top, weights + (size_t)t * top, lane,
                    mode, weight_scale);
}

extern "C" int ullm_moe_route(const float* logits, int ld, const float* correction, int T_, int n_router, int top,
                              int* ids, float* weights, int mode, float weight_scale, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (n_router < 1 || n_router > MOE_MAX_ROUTER || top < 1 || top > MOE_MAX_TOP || top > n_router || ld < n_router)
    return ULLM_ERR_SHAPE;
  if (mode < ROUTE_SOFTMAX_ALL || mode > ROUTE_SIGMOID) return ULLM_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(moe_route_kernel, dim3(T_), dim3(64), 0, stream, logits, ld, correction, n_router, top, ids, weights,
                     mode, weight_scale);
  ULLM_LAUNCH_CHECK();
}

// The router's product and the routing in one kernel: a block takes TPB tokens; their rows lie in shared memory as
// 32-bit values, every wave takes four router outputs at a time with four 16-byte pieces of each of their rows a
// lane under way (the loop is a chain of trips to memory otherwise), and every piece fetched serves all the block's
// tokens (four tokens and four waves a block for many tokens; one token and sixteen waves for few).  A lane adds a token's pieces in rising order, then the wave adds up: an order that depends on nothing but
// the row.  Then wave v routes token v.  The router's matrix is 32-bit [n_router, H].
template <typename T, int TPB>
__global__ void __launch_bounds__(TPB == 1 ? 1024 : 256)
moe_router_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ correction,
                  int n_tokens, int H, int n_router, int top, int* __restrict__ ids, float* __restrict__ weights, int mode,
                  float weight_scale) {
  extern __shared__ __attribute__((aligned(16))) float xrow[];          // [TPB][H]
  constexpr int RCAP = TPB == 1 ? MOE_MAX_ROUTER : 256;                // router outputs the variant takes
  __shared__ float z[TPB][RCAP], s_choice[TPB][RCAP];
  __shared__ float s_pick[TPB][MOE_MAX_TOP];
  const int t0 = blockIdx.x * TPB, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
  for (int q = 0; q < TPB; ++q) {
    const T* xr = x + (size_t)(t0 + q < n_tokens ? t0 + q : n_tokens - 1) * ldx;
    for (int i = tid; i < H; i += (int)blockDim.x) xrow[q * H + i] = ld_f32(xr + i);
  }
  __syncthreads();
  const bool vec = (H & 3) == 0 && (((uintptr_t)w) & 15) == 0;
  for (int e0 = 4 * wave; e0 < n_router; e0 += (int)(blockDim.x >> 4)) {
    float a[TPB][4];
#pragma unroll
    for (int q = 0; q < TPB; ++q)
#pragma unroll
      for (int u = 0; u < 4; ++u) a[q][u] = 0.f;
    const float* we[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) we[u] = w + (size_t)(e0 + u < n_router ? e0 + u : n_router - 1) * H;
    if (vec) {
      const int pieces = H >> 2;
      for (int p0 = lane; p0 < pieces; p0 += 256) {
        float4 wv[4][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int pj = p0 + 64 * j < pieces ? p0 + 64 * j : pieces - 1;
#pragma unroll
          for (int u = 0; u < 4; ++u) wv[u][j] = *reinterpret_cast<const float4*>(we[u] + 4 * pj);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (p0 + 64 * j >= pieces) break;
#pragma unroll
          for (int q = 0; q < TPB; ++q) {
            const float4 xv = *reinterpret_cast<const float4*>(xrow + q * H + 4 * (p0 + 64 * j));
#pragma unroll
            for (int u = 0; u < 4; ++u)
              a[q][u] = fmaf(xv.w, wv[u][j].w, fmaf(xv.z, wv[u][j].z, fmaf(xv.y, wv[u][j].y, fmaf(xv.x, wv[u][j].x, a[q][u]))));
          }
        }
      }
    } else {
      for (int i = lane; i < H; i += 64) {
#pragma unroll
        for (int q = 0; q < TPB; ++q)
#pragma unroll
          for (int u = 0; u < 4; ++u) a[q][u] = fmaf(xrow[q * H + i], we[u][i], a[q][u]);
      }
    }
#pragma unroll
    for (int q = 0; q < TPB; ++q)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float sum = wave_sum(a[q][u]);
        if (lane == 0 && e0 + u < n_router) z[q][e0 + u] = sum;
      }
  }
  __syncthreads();
  if (wave < TPB && t0 + wave < n_tokens)
    route_from_logits(z[wave], s_choice[wave], s_pick[wave], correction, n_router, top, ids + (size_t)(t0 + wave) * top,
                      weights + (size_t)(t0 + wave) * top, lane, mode, weight_scale);
}

extern "C" int ullm_moe_router(const void* x, int ldx, const float* w, const float* correction, int T_, int H,
                               int n_router, int top, int* ids, float* weights, int mode, float weight_scale, int dtype,
                               hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (mode < ROUTE_SOFTMAX_ALL || mode > ROUTE_SIGMOID) return ULLM_ERR_UNSUPPORTED;
  if (n_router < 1 || n_router > MOE_MAX_ROUTER || top < 1 || top > MOE_MAX_TOP || top > n_router || H < 1 || ldx < H ||
      (size_t)H * sizeof(float) > 48 * 1024)
    return ULLM_ERR_SHAPE;
  // many tokens: four a block, so that a piece of the router's matrix is fetched once for four rows (where their rows
  // and four sets of scores fit shared memory); few: a block each
  const bool four = T_ >= 512 && (size_t)H * sizeof(float) <= 8 * 1024 && n_router <= 256;
  const size_t lds = (size_t)H * sizeof(float) * (four ? 4 : 1);
  // a token a block: sixteen waves, so that up to 64 router outputs are summed in one round of trips to memory
  dim3 grid(four ? (T_ + 3) / 4 : T_), block(four ? 256 : 1024);
#define GO(TT, N) hipLaunchKernelGGL((moe_router_kernel<TT, N>), grid, block, lds, stream, (const TT*)x, ldx, w, correction, T_, H, \
    n_router, top, ids, weights, mode, weight_scale)
  if (dtype == ULLM_F32) { if (four) GO(float, 4); else GO(float, 1); }
  else if (dtype == ULLM_BF16) { if (four) GO(bf16_t, 4); else GO(bf16_t, 1); }
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------- grouping by expert
// One block.  offsets [experts + 1]; slot_of_pair [pairs] (-1: the pair's expert has no weights); token_of_slot [pairs];
// tiles [max_tiles + 1][3] = (expert, first slot, rows), rows 0 for the tiles no expert filled; the entry behind the
// list holds the number of tiles in use.
__global__ void __launch_bounds__(1024)
moe_sort_kernel(const int* __restrict__ ids, int n_pairs, int top, int n_experts, int tile_rows,
                int* __restrict__ offsets, int* __restrict__ slot_of_pair, int* __restrict__ token_of_slot,
                int* __restrict__ tiles, int max_tiles) {
  __shared__ int count[MOE_MAX_ROUTER], start[MOE_MAX_ROUTER + 1], cursor[MOE_MAX_ROUTER], tile_base[MOE_MAX_ROUTER + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < n_experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = tid; p < n_pairs; p += blockDim.x) {
    const int e = ids[p];
    if (e >= 0 && e < n_experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int off = 0, tb = 0;
    for (int e = 0; e < n_experts; ++e) {
      start[e] = off;
      cursor[e] = off;
      tile_base[e] = tb;
      off += count[e];
      tb += (count[e] + tile_rows - 1) / tile_rows;
    }
    start[n_experts] = off;
    tile_base[n_experts] = tb;
  }
  __syncthreads();
  for (int e = tid; e <= n_experts; e += blockDim.x) offsets[e] = start[e];
  for (int p = tid; p < n_pairs; p += blockDim.x) {
    const int e = ids[p];
    int slot = -1;
    if (e >= 0 && e < n_experts) {
      slot = atomicAdd(&cursor[e], 1);
      token_of_slot[slot] = p / top;
    }
    slot_of_pair[p] = slot;
  }
  for (int e = tid; e < n_experts; e += blockDim.x) {
    const int first = tile_base[e], n = tile_base[e + 1] - first;
    for (int i = 0; i < n && first + i < max_tiles; ++i) {
      const int left = count[e] - i * tile_rows;
      tiles[3 * (first + i)] = e;
      tiles[3 * (first + i) + 1] = start[e] + i * tile_rows;
      tiles[3 * (first + i) + 2] = left < tile_rows ? left : tile_rows;
    }
  }
  for (int i = tile_base[n_experts] + tid; i < max_tiles; i += blockDim.x) {
    tiles[3 * i] = 0;
    tiles[3 * i + 1] = 0;
    tiles[3 * i + 2] = 0;
  }
  if (tid == 0) {                                         // one more entry behind the list: how many tiles are in use
    tiles[3 * max_tiles] = tile_base[n_experts] < max_tiles ? tile_base[n_experts] : max_tiles;
    tiles[3 * max_tiles + 1] = 0;
    tiles[3 * max_tiles + 2] = 0;
  }
}

extern "C" int ullm_moe_sort(const int* ids, int n_pairs, int top, int n_experts, int tile_rows, int* offsets,
                             int* slot_of_pair, int* token_of_slot, int* tiles, int max_tiles, hipStream_t stream) {
  if (n_pairs <= 0) return 0;
  if (n_experts < 1 || n_experts > MOE_MAX_ROUTER || top < 1 || tile_rows < 1 || max_tiles < 1) return ULLM_ERR_SHAPE;
  // every routing fits: sum over experts of ceil(count / tile_rows) <= pairs / tile_rows + experts in use
  const long long most = (long long)n_pairs / tile_rows + (n_experts < n_pairs ? n_experts : n_pairs);
  if (max_tiles < most) return ULLM_ERR_SHAPE;
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, n_pairs, top, n_experts, tile_rows, offsets,
                     slot_of_pair, token_of_slot, tiles, max_tiles);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------- the clamped gated unit
// limit <= 0: the plain gated unit silu(g) * u.
template <bool EXACT>
__device__ __forceinline__ float moe_glu(float g, float u, float limit, float alpha) {
  if (limit <= 0.f)
    return (EXACT ? g / (1.f + expf(-g)) : fast_silu(g)) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  const float sg = EXACT ? 1.f / (1.f + expf(-alpha * g))
                         : __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.4426950408889634f * alpha * g));
  return g * sg * (u + 1.f);
}

// ------------------------------------------------------------------------------- products, one wave per value
// grid (tiles, column blocks); a block of 4 waves takes one tile's rows in turn, the row of x in shared memory,
// and each wave its share of the block's columns: lanes stride K, then the wave adds up (a fixed order).
template <typename T, bool GATED>
__global__ void __launch_bounds__(256)
moe_rows_simple_kernel(const T* __restrict__ x, int ldx, const int* __restrict__ row_index,
                       const T* __restrict__ w, const int* __restrict__ tiles, void* __restrict__ out_, int ldo,
                       int n_out, int K, int cols_per_block, float limit, float alpha) {
  extern __shared__ float xrow[];
  const int tile = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int e = tiles[3 * tile], slot0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  if (rows <= 0) return;
  const int c0 = blockIdx.y * cols_per_block;
  const int c1 = c0 + cols_per_block < n_out ? c0 + cols_per_block : n_out;
  const size_t w_rows = GATED ? 2 * (size_t)n_out : (size_t)n_out;
  const T* we = w + (size_t)e * w_rows * K;
  for (int r = 0; r < rows; ++r) {
    const int slot = slot0 + r;
    const T* xr = x + (size_t)(row_index ? row_index[slot] : slot) * ldx;
    __syncthreads();
    for (int i = tid; i < K; i += 256) xrow[i] = ld_f32(xr + i);
    __syncthreads();
    for (int c = c0 + wave; c < c1; c += 4) {
      const T* wg = we + (size_t)c * K;
      float a = 0.f, b = 0.f;
      for (int i = lane; i < K; i += 64) {
        a = fmaf(xrow[i], ld_f32(wg + i), a);
        if (GATED) b = fmaf(xrow[i], ld_f32(wg + (size_t)n_out * K + i), b);
      }
      a = wave_sum(a);
      if (GATED) b = wave_sum(b);
      if (lane == 0) {
        if (GATED) st_f32(reinterpret_cast<T*>(out_) + (size_t)slot * ldo + c, moe_glu<sizeof(T) == 4>(a, b, limit, alpha));
        else reinterpret_cast<float*>(out_)[(size_t)slot * ldo + c] = a;
      }
    }
  }
}

// ------------------------------------------------------------------------------- products on the matrix cores
// Few rows a tile (single tokens of a step): grid (tiles, groups of 16 output columns); tile = up to 16 * MT grouped
// rows of one expert.  The block's four waves share the 16 columns (GATED: the 16 gate rows and the 16 up rows of
// those columns) and take every fourth step of 64 along K, two steps of 32 in flight each; their sums are added
// through shared memory in wave order.  The work is streaming the chosen experts' matrices once, so it is cut into
// many blocks with many loads under way.  No load stands under a condition: a row past the tile's reads its last
// row, a column past the end the last column, a piece past the end of K the row's last piece (and is replaced by
// zeros); none is stored.
template <int MT, bool GATED>
__global__ void __launch_bounds__(256)
moe_rows_mfma_kernel(const bf16_t* __restrict__ x, int ldx, const int* __restrict__ row_index,
                     const bf16_t* __restrict__ w, const int* __restrict__ tiles, void* __restrict__ out_, int ldo,
                     int n_out, int K, float limit, float alpha) {
  constexpr int VALS = (GATED ? 8 : 4) * MT;
  __shared__ float part[3][VALS][64];
  const int tile = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int e = tiles[3 * tile], slot0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  if (rows <= 0) return;
  const int n0 = blockIdx.y * 16;
  const size_t w_rows = GATED ? 2 * (size_t)n_out : (size_t)n_out;
  const int wrow = n0 + r < n_out ? n0 + r : n_out - 1;
  const bf16_t* wg = w + ((size_t)e * w_rows + wrow) * K;
  const bf16_t* wu = wg + (size_t)n_out * K;
  const bf16_t* xr[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = 16 * t + r < rows ? 16 * t + r : rows - 1;
    xr[t] = x + (size_t)(row_index ? row_index[slot0 + row] : slot0 + row) * ldx;
  }
  f32x4_t acc_g[MT], acc_u[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    acc_g[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    acc_u[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const int last_piece = K - 8;                          // K is a multiple of 8
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  for (int k0 = 64 * wave; k0 < K; k0 += 256) {
    Pack8 a_g[2], a_u[2], b[2][MT];
    bool in[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int k = k0 + 32 * s + 8 * g;
      in[s] = k <= last_piece;
      const int kk = in[s] ? k : last_piece;
      a_g[s].u4 = ld_stream16(wg + kk);
      if (GATED) a_u[s].u4 = ld_stream16(wu + kk);
#pragma unroll
      for (int t = 0; t < MT; ++t) b[s][t].u4 = ld16(xr[t] + kk);
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (!in[s]) b[s][t].u4 = zero;
        acc_g[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_g[s].v, b[s][t].v, acc_g[t], 0, 0, 0);
        if (GATED) acc_u[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_u[s].v, b[s][t].v, acc_u[t], 0, 0, 0);
      }
    }
  }
  // the waves' sums, added in wave order
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        part[wave - 1][(GATED ? 8 : 4) * t + i][lane] = acc_g[t][i];
        if (GATED) part[wave - 1][8 * t + 4 + i][lane] = acc_u[t][i];
      }
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int v = 0; v < 3; ++v)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc_g[t][i] += part[v][(GATED ? 8 : 4) * t + i][lane];
        if (GATED) acc_u[t][i] += part[v][8 * t + 4 + i][lane];
      }
  // lane (r, g): row r of each 16-row group, columns n0 + 4g .. + 4
  const int c = n0 + 4 * g;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = 16 * t + r;
    if (row >= rows) continue;
    const size_t at = (size_t)(slot0 + row) * ldo + c;
    if (GATED) {
      bf16_t* o = reinterpret_cast<bf16_t*>(out_) + at;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = moe_glu<false>(acc_g[t][i], acc_u[t][i], limit, alpha);
      if (c + 3 < n_out && (ldo & 3) == 0) {
        *reinterpret_cast<uint2*>(o) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (c + i < n_out) o[i] = f32_to_bf16_bits(v[i]);
      }
    } else {
      float* o = reinterpret_cast<float*>(out_) + at;
      if (c + 3 < n_out && (ldo & 3) == 0) {
        *reinterpret_cast<float4*>(o) = make_float4(acc_g[t][0], acc_g[t][1], acc_g[t][2], acc_g[t][3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (c + i < n_out) o[i] = acc_g[t][i];
      }
    }
  }
}

// Many rows a tile (prompt portions): a block per (tile, 128 rows of the expert's matrix); tile = up to 16 MT = 64 or 128
// grouped rows of one expert.  A stage is 64 values of K: the tile's rows of x and 128 rows of the matrix (GATED: the
// gate rows and the up rows of 64 output columns; else 128 output columns) go through shared memory once a block,
// 128-byte rows whose 16-byte piece c of row r lies at piece c ^ ((r >> 1) & 7) (the 16 lanes the hardware serves
// together then read 16 different bank groups); the next stage is fetched into registers while the products of this
// one run.  Wave v takes matrix rows 16 v .. and 64 + 16 v .. (GATED: gate and up of the same columns) against all
// rows of x: 16 products per 12 reads of shared memory at 64 rows, 32 per 20 at 128 (and 64 rather than 43 products
// per byte fetched).
template <int MT, bool GATED>
__global__ void __launch_bounds__(256)
moe_tiles_mfma_kernel(const bf16_t* __restrict__ x, int ldx, const int* __restrict__ row_index,
                      const bf16_t* __restrict__ w, const int* __restrict__ tiles, int n_tiles, int n_col_blocks,
                      void* __restrict__ out_, int ldo, int n_out, int K, float limit, float alpha) {
  extern __shared__ __attribute__((aligned(16))) unsigned char tile_stages[];  // two stages take turns: x, then the matrix
  constexpr int XB = 16 * MT * 128, WB = 128 * 128;
  unsigned char* const xs2[2] = {tile_stages, tile_stages + XB + WB};
  unsigned char* const ws2[2] = {tile_stages + XB, tile_stages + 2 * XB + WB};
  // Workgroups go to the chip's 8 dies round-robin by their id and every die has a second-level cache of its own:
  // die d takes the d-th eighth of the tiles in use, tile by tile in the list's order with all of a tile's column
  // blocks side by side.  What runs on a die at one time is then a few tiles of one or two experts: a tile's rows
  // of x are fetched once for all its column blocks, an expert's matrix once for all its tiles.
  const int used = tiles[3 * n_tiles];
  const int total = used * n_col_blocks, per_die = (total + 7) / 8;
  const int item = ((int)blockIdx.x & 7) * per_die + ((int)blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per_die || item >= total) return;
  const int tile = item / n_col_blocks, col_block = item % n_col_blocks;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
  const int e = tiles[3 * tile], slot0 = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  if (rows <= 0) return;
  const int cols = GATED ? 64 : 128;                      // output columns of a block
  const int n0 = col_block * cols;
  const size_t w_rows = GATED ? 2 * (size_t)n_out : (size_t)n_out;
  const bf16_t* we = w + (size_t)e * w_rows * K;
  // what this thread fetches of a stage: piece `pc` of x rows prow + 32 i and of matrix rows prow + 32 i
  constexpr int XP = MT / 2;                              // pieces of x a thread fetches a stage
  const int pc = tid & 7, prow = tid >> 3;
  const bf16_t* xsrc[XP];
  const bf16_t* wsrc[4];
  int xput[XP], wput[4];
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const int row = prow + 32 * i, rr = row < rows ? row : rows - 1;
    xsrc[i] = x + (size_t)(row_index ? row_index[slot0 + rr] : slot0 + rr) * ldx;
    xput[i] = row * 128 + ((pc ^ ((row >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = prow + 32 * i;                       // 0 .. 127 of the block's matrix rows
    int n = GATED ? n0 + (row & 63) : n0 + row;
    if (n >= n_out) n = n_out - 1;
    wsrc[i] = we + ((GATED && row >= 64 ? (size_t)n_out : 0) + n) * K;
    wput[i] = row * 128 + ((pc ^ ((row >> 1) & 7)) << 4);
  }
  const int last_piece = K - 8;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  // two sets of registers: a stage is fetched two stages before its products, written to shared memory one before
  uint4 xreg[2][XP], wreg[2][4];
  auto fetch = [&](int set, int k0) __attribute__((always_inline)) {
    const int k = k0 + 8 * pc;
    const bool in = k <= last_piece;
    const int kk = in ? k : last_piece;
#pragma unroll
    for (int i = 0; i < XP; ++i) xreg[set][i] = ld16(xsrc[i] + kk);
#pragma unroll
    for (int i = 0; i < 4; ++i) wreg[set][i] = ld16(wsrc[i] + kk);    // the expert's other tiles read the same rows: cached
    if (!in) {
#pragma unroll
      for (int i = 0; i < XP; ++i) xreg[set][i] = zero;
    }
  };
  auto put = [&](int set, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < XP; ++i) st16(xs2[buf] + xput[i], xreg[set][i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) st16(ws2[buf] + wput[i], wreg[set][i]);
  };
  f32x4_t acc[2][MT];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[h][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  auto products = [&](int buf) __attribute__((always_inline)) {
    const unsigned char* xs = xs2[buf];
    const unsigned char* ws = ws2[buf];
    // both steps of 32 are read before the first product: the second step's reads travel during the first's products
    Pack8 a[2][2], b[2][MT];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = 64 * h + 16 * wave + r;
        a[s][h].u4 = ld16(ws + row * 128 + (((4 * s + g) ^ ((row >> 1) & 7)) << 4));
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int row = 16 * t + r;
        b[s][t].u4 = ld16(xs + row * 128 + (((4 * s + g) ^ ((row >> 1) & 7)) << 4));
      }
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][h].v, b[s][t].v, acc[h][t], 0, 0, 0);
  };
  // No fetch stands under a condition (the compiler then waits for every load under way at the next use of any): a
  // stage past the end of K reads the rows' last pieces again and is never written to shared memory.
  fetch(0, 0);
  put(0, 0);
  __syncthreads();
  fetch(0, 64);
  for (int k0 = 0; k0 < K; k0 += 128) {
    // stage k0 lies in buffer 0, set 0 holds stage k0 + 64 (on its way)
    fetch(1, k0 + 128);
    products(0);
    if (k0 + 64 < K) put(0, 1);          // buffer 1 was last read before the barrier that ended the step before
    __syncthreads();
    if (k0 + 64 >= K) break;
    // stage k0 + 64 lies in buffer 1, set 1 holds stage k0 + 128
    fetch(0, k0 + 192);
    products(1);
    if (k0 + 128 < K) put(1, 0);
    __syncthreads();
  }
  // lane (r, g): row r of each 16-row group; columns 16 wave + 4g .. + 4 of the block's (and 64 further on)
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = 16 * t + r;
    if (row >= rows) continue;
    if (GATED) {
      const int c = n0 + 16 * wave + 4 * g;
      bf16_t* o = reinterpret_cast<bf16_t*>(out_) + (size_t)(slot0 + row) * ldo + c;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = moe_glu<false>(acc[0][t][i], acc[1][t][i], limit, alpha);
      if (c + 3 < n_out && (ldo & 3) == 0) {
        *reinterpret_cast<uint2*>(o) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (c + i < n_out) o[i] = f32_to_bf16_bits(v[i]);
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int c = n0 + 64 * h + 16 * wave + 4 * g;
        float* o = reinterpret_cast<float*>(out_) + (size_t)(slot0 + row) * ldo + c;
        if (c + 3 < n_out && (ldo & 3) == 0) {
          *reinterpret_cast<float4*>(o) = make_float4(acc[h][t][0], acc[h][t][1], acc[h][t][2], acc[h][t][3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (c + i < n_out) o[i] = acc[h][t][i];
        }
      }
    }
  }
}

// Rows of a tile the matrix-core kernels take for a launch made with `tile_rows` rows a tile.
extern "C" int ullm_moe_mfma_supports(int K, int ldx, int tile_rows) {
  return K >= 8 && K % 8 == 0 && ldx % 8 == 0 && (tile_rows == 16 || tile_rows == 32 || tile_rows == 64 || tile_rows == 128);
}

template <int MT, bool GATED, typename... Args>
static void launch_tiles(dim3 grid, hipStream_t stream, Args... args) {
  constexpr int bytes = 2 * (16 * MT * 128 + 128 * 128);
  static const hipError_t allowed = hipFuncSetAttribute((const void*)moe_tiles_mfma_kernel<MT, GATED>,
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  (void)allowed;
  hipLaunchKernelGGL((moe_tiles_mfma_kernel<MT, GATED>), grid, dim3(256), bytes, stream, args...);
}

// out[slot] = glu(x[row_index[slot]] Wg^T, x Wu^T) (gated: out in x's dtype, w [experts, 2 n_out, K]) or
// x[slot] W^T (not gated: out float32, w [experts, n_out, K]) over the tiles' rows.  row_index may be null.
extern "C" int ullm_moe_rows(const void* x, int ldx, const int* row_index, const void* w, const int* tiles,
                             int max_tiles, int tile_rows, void* out, int ldo, int n_out, int K, int gated,
                             float limit, float alpha, int dtype, hipStream_t stream) {
  if (max_tiles <= 0) return 0;
  if (n_out < 1 || K < 1 || ldx < K || ldo < n_out || tile_rows < 1) return ULLM_ERR_SHAPE;
  if (dtype == ULLM_BF16 && ullm_moe_mfma_supports(K, ldx, tile_rows) && !((uintptr_t)x & 15) && !((uintptr_t)w & 15)) {
    if (tile_rows >= 64) {
      const int col_blocks = (n_out + (gated ? 63 : 127)) / (gated ? 64 : 128);
      const long long total = (long long)max_tiles * col_blocks;
      if (total > 0x3fffffffLL) return ULLM_ERR_SHAPE;
      dim3 grid((unsigned)(8 * ((total + 7) / 8)));
#define TILES(MT, G) launch_tiles<MT, G>(grid, stream, (const bf16_t*)x, ldx, row_index, (const bf16_t*)w, tiles, max_tiles, \
    col_blocks, out, ldo, n_out, K, limit, alpha)
      if (tile_rows == 64) { if (gated) TILES(4, true); else TILES(4, false); }
      else { if (gated) TILES(8, true); else TILES(8, false); }
#undef TILES
      ULLM_LAUNCH_CHECK();
    }
    dim3 grid(max_tiles, (n_out + 15) / 16), block(256);
    if (grid.y > 65535) return ULLM_ERR_SHAPE;
#define GO(MT, G) hipLaunchKernelGGL((moe_rows_mfma_kernel<MT, G>), grid, block, 0, stream, (const bf16_t*)x, ldx, row_index, \
    (const bf16_t*)w, tiles, out, ldo, n_out, K, limit, alpha)
    if (tile_rows == 16) { if (gated) GO(1, true); else GO(1, false); }
    else { if (gated) GO(2, true); else GO(2, false); }
#undef GO
    ULLM_LAUNCH_CHECK();
  }
  if ((size_t)K * sizeof(float) > 64 * 1024) return ULLM_ERR_SHAPE;
  const int cols_per_block = 64;
  dim3 grid(max_tiles, (n_out + cols_per_block - 1) / cols_per_block), block(256);
  if (grid.y > 65535) return ULLM_ERR_SHAPE;
  const size_t lds = (size_t)K * sizeof(float);
#define GO(TT, G) hipLaunchKernelGGL((moe_rows_simple_kernel<TT, G>), grid, block, lds, stream, (const TT*)x, ldx, row_index, \
    (const TT*)w, tiles, out, ldo, n_out, K, cols_per_block, limit, alpha)
  if (dtype == ULLM_F32) { if (gated) GO(float, true); else GO(float, false); }
  else if (dtype == ULLM_BF16) { if (gated) GO(bf16_t, true); else GO(bf16_t, false); }
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------- the weighted sum
// out[t][c] = base[t][c] + bias[c] + shared[t][c] + sum_k weights[t][k] * (ids[t][k] < n_experts ? y[slot][c] : x[t][c]);
// base (float32 or TX), bias (float32), shared (TX) may be null.  grid (tokens, groups of columns): a thread takes
// VEC consecutive columns, all its loads independent of each other.
template <typename TX, typename TB, int VEC>
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ y, const TX* __restrict__ x, int ldx, const int* __restrict__ ids,
                   const float* __restrict__ weights, const int* __restrict__ slot_of_pair, int top, int n_experts,
                   const TB* __restrict__ base, const float* __restrict__ bias, const TX* __restrict__ shared,
                   float* __restrict__ out, int H) {
  const int t = blockIdx.x, c = VEC * (blockIdx.y * 256 + threadIdx.x);
  if (c >= H) return;
  float a[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    a[i] = base ? ld_f32(base + (size_t)t * H + c + i) : 0.f;
    if (bias) a[i] += bias[c + i];
    if (shared) a[i] += ld_f32(shared + (size_t)t * H + c + i);
  }
  for (int k = 0; k < top; ++k) {
    const int e = ids[(size_t)t * top + k];
    const float wk = weights[(size_t)t * top + k];
    if (e < n_experts) {
      const float* yr = y + (size_t)slot_of_pair[(size_t)t * top + k] * H + c;
#pragma unroll
      for (int i = 0; i < VEC; ++i) a[i] = fmaf(wk, yr[i], a[i]);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) a[i] = fmaf(wk, ld_f32(x + (size_t)t * ldx + c + i), a[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < VEC; ++i) out[(size_t)t * H + c + i] = a[i];
}

extern "C" int ullm_moe_combine(const float* y, const void* x, int ldx, const int* ids, const float* weights,
                                const int* slot_of_pair, int top, int n_experts, const void* base, int base_dtype,
                                const float* bias, const void* shared, float* out, int T_, int H, int dtype,
                                hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (H < 1 || top < 1 || ldx < H) return ULLM_ERR_SHAPE;
  const int vec = H % 4 == 0 ? 4 : 1;
  dim3 grid(T_, (H / vec + 255) / 256), block(256);
  if (grid.y > 65535) return ULLM_ERR_SHAPE;
#define GO(TX, TB, V) hipLaunchKernelGGL((moe_combine_kernel<TX, TB, V>), grid, block, 0, stream, y, (const TX*)x, ldx, ids, weights, \
    slot_of_pair, top, n_experts, (const TB*)base, bias, (const TX*)shared, out, H)
#define GOV(TX, TB) do { if (vec == 4) GO(TX, TB, 4); else GO(TX, TB, 1); } while (0)
  if (dtype == ULLM_F32) {
    if (base && base_dtype != ULLM_F32) return ULLM_ERR_DTYPE;
    GOV(float, float);
  } else if (dtype == ULLM_BF16) {
    if (base && base_dtype == ULLM_BF16) GOV(bf16_t, bf16_t);
    else GOV(bf16_t, float);
  } else {
    return ULLM_ERR_DTYPE;
  }
#undef GOV
#undef GO
  ULLM_LAUNCH_CHECK();
}
