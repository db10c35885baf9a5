// Linear recurrences with a matrix state per head that decays per key channel, and what stands around them.
//
//   state   S [N, P] per head (N key channels, P value channels), float32, carried per request in a state row
//   update  S_t = diag(d_t) S_(t-1) + k_t v_t^T
//   output  after the update (o_t = S_t^T q_t), or before it with a bonus for the current token
//           (o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t)
//   decay   d_t[n] is one constant per head, or sigmoid(z)^(1/tau), or exp(-exp(z)) of a raw value z[t, head, n]
//   inputs  q, k, v are float32 rows (columns of projections), optionally through silu, q times a constant
//
// Around it: the blend of a token's input with the previous token's (`token shift`), whose last row is part of the
// request's state, and the norm of the outputs (per head or over all heads) times a gain and a gate.
// A batch is any mix of prompt portions and single tokens: entry b owns tokens q_start[b] .. q_start[b+1]-1 and the
// state row entry_slot[b]; rows of requests that start at their first token are zero when a step begins.
// Everything is 32-bit.  A state element goes through the same operations in the same order wherever a prompt is
// cut, and a token's output sums its partial sums in a fixed order.
#include "common.h"

enum { DECAY_PER_HEAD = 0, DECAY_SIGMOID_ROOT = 1, DECAY_EXP_EXP = 2 };
enum { GATE_SILU = 0, GATE_SIGMOID = 1 };

#define SCAN_THREADS 256
#define SCAN_CHUNK 16

__device__ __forceinline__ float exact_silu(float z) { return z / (1.f + expf(-z)); }

// The decay of a raw value.  sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau), with softplus(x) = max(x, 0) + log1p(e^-|x|).
__device__ __forceinline__ float decay_of(float z, int kind, float inv_tau) {
  if (kind == DECAY_SIGMOID_ROOT) {
    const float x = -z;
    const float sp = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
    return expf(-sp * inv_tau);
  }
  return expf(-expf(z));
}

// A barrier for shared memory alone: loads and stores of global memory stay in flight.
__device__ __forceinline__ void shared_memory_barrier() {
#ifdef __HIP_DEVICE_COMPILE__
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#endif
}

struct ScanArgs {
  const float* q;
  const float* k;
  const float* v;
  const float* z;           // raw decays [T, heads * N] (stride z_ld) or, DECAY_PER_HEAD, the heads' constants
  const float* bonus;       // [heads, N] or null
  float* state;
  long long state_stride, state_off;
  const int* q_start;
  const int* entry_slot;
  float* out;               // [T, heads * P]
  int q_ld, k_ld, v_ld, z_ld;
  int heads, N, P;
  int decay_kind, silu_inputs, before, write_state;
  float q_scale, inv_tau;
};

// One block per (entry, head, slice of PC value channels).  Thread (r, p) keeps the NPT state rows n = r * NPT ..
// of column p in registers; R = 256 / PC such threads cover R * NPT >= N rows (rows from N on see k = q = 0).  The
// entry's tokens are walked in chunks of SCAN_CHUNK: the chunk's q, k, decays and v are staged in shared memory
// (activation, scale and the decay's function applied once on the way), the next chunk's raw values are fetched
// into registers before the current chunk is worked on and written to the other buffer afterwards.  Every thread
// leaves one partial sum per token; after one barrier the block adds each token's R partial sums in the order of r.
template <int PC, int NPT, bool BEFORE>
__global__ void __launch_bounds__(SCAN_THREADS)
decay_scan_kernel(const ScanArgs a) {
  constexpr int R = SCAN_THREADS / PC;
  constexpr int NP = R * NPT;                       // padded key channels
  constexpr int ROW = 3 * NP + PC;                  // staged values of a token: q | k | d | v
  constexpr int PER_BUF = SCAN_CHUNK * ROW;
  constexpr int PER_TOK = (3 * NP + PC + 15) / 16;  // values each of a token's 16 staging lanes brings
  extern __shared__ __attribute__((aligned(16))) float shared[];
  float* part = shared + 2 * PER_BUF;               // [chunk][R][PC]
  const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * PC;
  const int tid = threadIdx.x, p = tid % PC, r = tid / PC;
  const int N = a.N, P = a.P;
  const bool column = p0 + p < P;
  const int first = a.q_start[b], end = a.q_start[b + 1];
  float* row = a.state + (size_t)a.entry_slot[b] * a.state_stride + a.state_off + (size_t)h * N * P + p0;
  float s[NPT], u[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int n = r * NPT + i;
    s[i] = (column && n < N) ? row[(size_t)n * P + p] : 0.f;
    u[i] = (BEFORE && a.bonus != nullptr && n < N) ? a.bonus[(size_t)h * N + n] : 0.f;
  }
  const float head_decay = a.decay_kind == DECAY_PER_HEAD ? a.z[h] : 1.f;
  const int tl = tid / 16, ln = tid % 16;           // staging: token of the chunk, lane of its 16
  float raw[PER_TOK];
  // element e of a token's staged row: [0, NP) q, [NP, 2NP) k, [2NP, 3NP) decay, then PC values of v
  auto fetch = [&](int c0) __attribute__((always_inline)) {
    const int tok = c0 + tl;
    const bool live = tok < end;
#pragma unroll
    for (int i = 0; i < PER_TOK; ++i) {
      const int e = ln + 16 * i;
      float val = 0.f;
      if (live && e < ROW) {
        if (e < 3 * NP) {
          const int which = e / NP, n = e % NP;
          if (n < N) {
            if (which == 0) val = a.q[(size_t)tok * a.q_ld + h * N + n];
            else if (which == 1) val = a.k[(size_t)tok * a.k_ld + h * N + n];
            else if (a.decay_kind != DECAY_PER_HEAD) val = a.z[(size_t)tok * a.z_ld + h * N + n];
          }
        } else if (p0 + e - 3 * NP < P) {
          val = a.v[(size_t)tok * a.v_ld + h * P + p0 + e - 3 * NP];
        }
      }
      raw[i] = val;
    }
  };
  auto put = [&](int c0, float* buf) __attribute__((always_inline)) {
    const bool live = c0 + tl < end;
    float* dst = buf + tl * ROW;
#pragma unroll
    for (int i = 0; i < PER_TOK; ++i) {
      const int e = ln + 16 * i;
      if (e < ROW) {
        float val = raw[i];
        const int which = e < 3 * NP ? e / NP : 3;
        if (which == 2) {
          // tokens past the entry's end and rows past N: decay 1 on a state that takes nothing
          val = (!live || e % NP >= N) ? 1.f : (a.decay_kind == DECAY_PER_HEAD ? head_decay : decay_of(val, a.decay_kind, a.inv_tau));
        } else {
          if (a.silu_inputs) val = exact_silu(val);
          if (which == 0) val *= a.q_scale;
        }
        dst[e] = val;
      }
    }
  };
  fetch(first);
  put(first, shared);
  shared_memory_barrier();
  int turn = 0;
  for (int c0 = first; c0 < end; c0 += SCAN_CHUNK) {
    const float* buf = shared + turn * PER_BUF;
    const bool more = c0 + SCAN_CHUNK < end;
    if (more) fetch(c0 + SCAN_CHUNK);
    const int n_tok = end - c0 < SCAN_CHUNK ? end - c0 : SCAN_CHUNK;
    for (int t = 0; t < n_tok; ++t) {
      const float* in = buf + t * ROW + r * NPT;
      const float vp = buf[t * ROW + 3 * NP + p];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NPT; ++i) {
        const float qn = in[i], kn = in[NP + i], dn = in[2 * NP + i];
        const float kv = kn * vp;
        if (BEFORE) {
          acc += (s[i] + u[i] * kv) * qn;
          s[i] = dn * s[i] + kv;
        } else {
          s[i] = dn * s[i] + kv;
          acc += s[i] * qn;
        }
      }
      part[(t * R + r) * PC + p] = acc;
    }
    shared_memory_barrier();
    for (int e = tid; e < n_tok * PC; e += SCAN_THREADS) {
      const int t = e / PC, pp = e % PC;
      if (p0 + pp < P) {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) sum += part[(t * R + i) * PC + pp];
        a.out[(size_t)(c0 + t) * a.heads * P + h * P + p0 + pp] = sum;
      }
    }
    if (more) put(c0 + SCAN_CHUNK, shared + (1 - turn) * PER_BUF);
    shared_memory_barrier();
    turn = 1 - turn;
  }
  if (a.write_state && column) {
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const int n = r * NPT + i;
      if (n < N) row[(size_t)n * P + p] = s[i];
    }
  }
}

template <int PC, int NPT>
static int launch_decay_scan(const ScanArgs& a, int B_, hipStream_t stream) {
  constexpr int R = SCAN_THREADS / PC, NP = R * NPT;
  constexpr size_t need = (2 * (size_t)SCAN_CHUNK * (3 * NP + PC) + (size_t)SCAN_CHUNK * R * PC) * sizeof(float);
  static_assert(need <= 160 * 1024, "a block's staging fits the shared memory of a compute unit");
  const dim3 grid(B_, a.heads, (a.P + PC - 1) / PC);
  if (a.before) {
    if (need > 48 * 1024) {
      const hipError_t e = hipFuncSetAttribute((const void*)decay_scan_kernel<PC, NPT, true>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)need);
      if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL((decay_scan_kernel<PC, NPT, true>), grid, dim3(SCAN_THREADS), need, stream, a);
  } else {
    if (need > 48 * 1024) {
      const hipError_t e = hipFuncSetAttribute((const void*)decay_scan_kernel<PC, NPT, false>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)need);
      if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL((decay_scan_kernel<PC, NPT, false>), grid, dim3(SCAN_THREADS), need, stream, a);
  }
  ULLM_LAUNCH_CHECK();
}

extern "C" int ullm_decay_scan(const float* q, int q_ld, const float* k, int k_ld, const float* v, int v_ld, const float* z,
                               int z_ld, int decay_kind, float tau, const float* bonus, int silu_inputs, float q_scale,
                               int before, float* state, long long state_stride, long long state_off,
                               const int* q_start, const int* entry_slot, float* out, int B_, int heads, int N, int P,
                               int write_state, hipStream_t stream) {
  if (B_ <= 0) return 0;
  if (heads <= 0 || N <= 0 || P <= 0 || N > 256) return ULLM_ERR_SHAPE;
  if (decay_kind < DECAY_PER_HEAD || decay_kind > DECAY_EXP_EXP || z == nullptr) return ULLM_ERR_UNSUPPORTED;
  if (decay_kind == DECAY_SIGMOID_ROOT && !(tau > 0.f)) return ULLM_ERR_UNSUPPORTED;
  ScanArgs a;
  a.q = q, a.k = k, a.v = v, a.z = z, a.bonus = bonus, a.state = state, a.state_stride = state_stride, a.state_off = state_off;
  a.q_start = q_start, a.entry_slot = entry_slot, a.out = out, a.q_ld = q_ld, a.k_ld = k_ld, a.v_ld = v_ld, a.z_ld = z_ld;
  a.heads = heads, a.N = N, a.P = P, a.decay_kind = decay_kind, a.silu_inputs = silu_inputs, a.before = before;
  a.write_state = write_state, a.q_scale = q_scale, a.inv_tau = decay_kind == DECAY_SIGMOID_ROOT ? 1.f / tau : 1.f;
#define SCAN_GO(PC, NPT) return launch_decay_scan<PC, NPT>(a, B_, stream)
  // whole rows of 64 value channels a block where there are blocks enough without slicing the heads (a step of
  // many requests: the state's rows then move as whole lines); else slices of 16
  if (P % 64 == 0 && N <= 128 && (long long)B_ * heads >= 1024) {
    if (N <= 32) SCAN_GO(64, 8);
    if (N <= 64) SCAN_GO(64, 16);
    SCAN_GO(64, 32);
  }
  if (N <= 16) SCAN_GO(16, 1);
  if (N <= 32) SCAN_GO(16, 2);
  if (N <= 64) SCAN_GO(16, 4);
  if (N <= 128) SCAN_GO(16, 8);
  SCAN_GO(16, 16);
#undef SCAN_GO
}

// ------------------------------------------------------------------ token shift
// out[m, t, :] = x[t] + (prev(t) - x[t]) * mu[m] for m < M, with prev(t) the row before t in its entry or, for an
// entry's first token, what the state row holds (the last row of the step before; zeros at a request's start).
// The block of an entry's first token then puts the entry's last row into the state row: a thread reads the old
// value of a column before it writes the new one.
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(const T* __restrict__ x, const float* __restrict__ mu, float* __restrict__ state,
                   long long state_stride, long long state_off, const int* __restrict__ token_entry,
                   const int* __restrict__ q_start, const int* __restrict__ entry_slot, T* __restrict__ out, int T_,
                   int H, int M, int write_state) {
  const int t = blockIdx.x;
  const int b = token_entry[t];
  const int first = q_start[b];
  const bool head = t == first;
  float* row = state + (size_t)entry_slot[b] * state_stride + state_off;
  const int last = q_start[b + 1] - 1;
  for (int col = threadIdx.x; col < H; col += 256) {
    const float cur = ld_f32(x + (size_t)t * H + col);
    const float prev = head ? row[col] : ld_f32(x + (size_t)(t - 1) * H + col);
    const float diff = prev - cur;
    for (int m = 0; m < M; ++m) st_f32(out + ((size_t)m * T_ + t) * H + col, cur + diff * mu[(size_t)m * H + col]);
    if (head && write_state) row[col] = ld_f32(x + (size_t)last * H + col);
  }
}

extern "C" int ullm_token_shift(const void* x, const float* mu, float* state, long long state_stride, long long state_off,
                                const int* token_entry, const int* q_start, const int* entry_slot, void* out, int T_,
                                int H, int M, int write_state, int dtype, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (H < 1 || M < 1) return ULLM_ERR_SHAPE;
  if (dtype == ULLM_F32)
    hipLaunchKernelGGL(token_shift_kernel<float>, dim3(T_), dim3(256), 0, stream, (const float*)x, mu, state, state_stride,
                       state_off, token_entry, q_start, entry_slot, (float*)out, T_, H, M, write_state);
  else if (dtype == ULLM_BF16)
    hipLaunchKernelGGL(token_shift_kernel<bf16_t>, dim3(T_), dim3(256), 0, stream, (const bf16_t*)x, mu, state, state_stride,
                       state_off, token_entry, q_start, entry_slot, (bf16_t*)out, T_, H, M, write_state);
  else return ULLM_ERR_DTYPE;
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ norm of the outputs, gain and gate
// The row o [width] is cut into `parts` equal parts (the heads, or one part); each is divided by its root mean
// square (eps inside the root), multiplied by gain[c % gain_len] (a gain per value channel shared by the heads, or
// one per column) and by silu or sigmoid of the gate's raw value g[t, c].  A wave per part, parts taken in turn.
template <typename TO>
__global__ void __launch_bounds__(256)
gated_unit_norm_kernel(const float* __restrict__ o, const float* __restrict__ g, int g_ld, const float* __restrict__ gain,
                       int gain_len, float eps, int gate_kind, TO* __restrict__ out, int width, int parts) {
  const int t = blockIdx.x, lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int size = width / parts;
  for (int part = wave; part < parts; part += 256 / WAVE) {
    const float* src = o + (size_t)t * width + (size_t)part * size;
    float sq = 0.f;
    for (int c = lane; c < size; c += WAVE) sq += src[c] * src[c];
    const float r = 1.f / sqrtf(wave_sum(sq) / (float)size + eps);
    for (int c = lane; c < size; c += WAVE) {
      const int col = part * size + c;
      const float z = g[(size_t)t * g_ld + col];
      const float gate = gate_kind == GATE_SIGMOID ? 1.f / (1.f + expf(-z)) : exact_silu(z);
      st_f32(out + (size_t)t * width + col, src[c] * r * gain[col % gain_len] * gate);
    }
  }
}

extern "C" int ullm_gated_unit_norm(const float* o, const float* g, int g_ld, const float* gain, int gain_len, float eps,
                                    int gate_kind, void* out, int T_, int width, int parts, int out_dtype,
                                    hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (width < 1 || parts < 1 || width % parts || gain_len < 1 || width % gain_len) return ULLM_ERR_SHAPE;
  if (gate_kind != GATE_SILU && gate_kind != GATE_SIGMOID) return ULLM_ERR_UNSUPPORTED;
  if (out_dtype == ULLM_F32)
    hipLaunchKernelGGL(gated_unit_norm_kernel<float>, dim3(T_), dim3(256), 0, stream, o, g, g_ld, gain, gain_len, eps,
                       gate_kind, (float*)out, width, parts);
  else if (out_dtype == ULLM_BF16)
    hipLaunchKernelGGL(gated_unit_norm_kernel<bf16_t>, dim3(T_), dim3(256), 0, stream, o, g, g_ld, gain, gain_len, eps,
                       gate_kind, (bf16_t*)out, width, parts);
  else return ULLM_ERR_DTYPE;
  ULLM_LAUNCH_CHECK();
}
