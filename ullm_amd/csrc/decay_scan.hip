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

enum { DECAY_PER_HEAD = 0, DECAY_SIGMOID_ROOT = 1, DECAY_EXP_EXP = 2, DECAY_READY = 3 };   // READY: z holds the decays themselves
typedef __attribute__((ext_vector_type(4))) float scan_f32x4;
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
// entry's tokens are walked in chunks of CH: the chunk's q, k, decays and v are staged in shared memory
// (activation, scale and the decay's function applied on the way unless a pass before has applied them), the next
// chunk's raw values are fetched into registers before the current chunk is worked on and written to the other
// buffer afterwards.  A token's staged values are read one to three tokens ahead of the arithmetic that uses them.  Every
// thread leaves one partial sum per token; after one barrier the block adds each token's R partial sums in the
// order of r.  CH = 1 serves steps of single tokens: little shared memory, so that many blocks of a compute unit
// have their state rows on the way at once.
template <int PC, int NPT, bool BEFORE, int CH, bool VEC = false>
__global__ void __launch_bounds__(SCAN_THREADS)
decay_scan_kernel(const ScanArgs a) {
  constexpr int R = SCAN_THREADS / PC;
  constexpr int NP = R * NPT;                       // padded key channels
  constexpr int ROW = 3 * NP + PC;                  // staged values of a token: q | k | d | v
  constexpr int PER_BUF = CH * ROW;
  constexpr int LANES = SCAN_THREADS / CH;          // staging lanes of a token
  constexpr int SV = VEC ? 4 : 1;                   // values a staging lane brings at once (VEC: 16-byte pieces)
  constexpr int PER_TOK = (ROW / SV + LANES - 1) / LANES;
  static_assert(!VEC || (NP % 4 == 0 && PC % 4 == 0), "16-byte pieces do not straddle q | k | d | v");
  extern __shared__ __attribute__((aligned(16))) float shared[];
  constexpr int PART = R * PC + (PC < 64 ? PC : 0);   // a token's partial sums, padded: the tokens of a wave's lanes in other banks
  float* part = shared + 2 * PER_BUF;               // [chunk][PART]
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
  const int tl = tid / LANES, ln = tid % LANES;     // staging: token of the chunk, lane of its LANES
  float raw[PER_TOK * SV];
  // element e of a token's staged row: [0, NP) q, [NP, 2NP) k, [2NP, 3NP) decay, then PC values of v
  auto fetch = [&](int c0) __attribute__((always_inline)) {
    const int tok = c0 + tl;
    const bool live = tok < end;
#pragma unroll
    for (int i = 0; i < PER_TOK; ++i) {
      const int e = SV * (ln + LANES * i);
      if constexpr (VEC || CH == 1) {
        // the address is chosen first and one load follows: the loads of a lane are all on their way before the
        // first is waited for (a step of single tokens is made of such waits).  (With 16-byte pieces N and P are
        // multiples of four: a piece lies inside its row or outside.)
        const float* src = nullptr;
        if (live && e < ROW) {
          if (e < 3 * NP) {
            const int which = e / NP, n = e % NP;
            if (n < N) {
              if (which == 0) src = a.q + (size_t)tok * a.q_ld + h * N + n;
              else if (which == 1) src = a.k + (size_t)tok * a.k_ld + h * N + n;
              else if (a.decay_kind != DECAY_PER_HEAD) src = a.z + (size_t)tok * a.z_ld + h * N + n;
            }
          } else if (p0 + e - 3 * NP < P) {
            src = a.v + (size_t)tok * a.v_ld + h * P + p0 + e - 3 * NP;
          }
        }
        if constexpr (VEC) {
          const scan_f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
          const scan_f32x4 val = src ? *reinterpret_cast<const scan_f32x4*>(src) : zero4;
          raw[4 * i] = val.x, raw[4 * i + 1] = val.y, raw[4 * i + 2] = val.z, raw[4 * i + 3] = val.w;
        } else {
          raw[i] = src ? *src : 0.f;
        }
      } else {
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
    }
  };
  auto put = [&](int c0, float* buf) __attribute__((always_inline)) {
    const bool live = c0 + tl < end;
    float* dst = buf + tl * ROW;
#pragma unroll
    for (int i = 0; i < PER_TOK; ++i) {
      const int e0 = SV * (ln + LANES * i);
      if (e0 < ROW) {
        const int which = e0 < 3 * NP ? e0 / NP : 3;
        float val[SV];
#pragma unroll
        for (int j = 0; j < SV; ++j) {
          float x = raw[SV * i + j];
          if (which == 2) {
            // tokens past the entry's end and rows past N: decay 1 on a state that takes nothing
            if (!live || (e0 + j) % NP >= N) x = 1.f;
            else if (a.decay_kind == DECAY_PER_HEAD) x = head_decay;
            else if (a.decay_kind != DECAY_READY) x = decay_of(x, a.decay_kind, a.inv_tau);
          } else {
            if (a.silu_inputs) x = exact_silu(x);
            if (which == 0) x *= a.q_scale;
          }
          val[j] = x;
        }
        if constexpr (VEC) {
          const scan_f32x4 v4 = {val[0], val[1], val[2], val[3]};
          *reinterpret_cast<scan_f32x4*>(dst + e0) = v4;
        } else {
          dst[e0] = val[0];
        }
      }
    }
  };
  struct TokenIn {
    float q[NPT], k[NPT], d[NPT];
    float v;
  };
  auto read_token = [&](const float* buf, int t, TokenIn& in) __attribute__((always_inline)) {
    const float* src = buf + t * ROW + r * NPT;
    if constexpr (NPT % 4 == 0) {
#pragma unroll
      for (int i = 0; i < NPT; i += 4) {
        const scan_f32x4 qq = *reinterpret_cast<const scan_f32x4*>(src + i);
        const scan_f32x4 kk = *reinterpret_cast<const scan_f32x4*>(src + NP + i);
        const scan_f32x4 dd = *reinterpret_cast<const scan_f32x4*>(src + 2 * NP + i);
        in.q[i] = qq.x, in.q[i + 1] = qq.y, in.q[i + 2] = qq.z, in.q[i + 3] = qq.w;
        in.k[i] = kk.x, in.k[i + 1] = kk.y, in.k[i + 2] = kk.z, in.k[i + 3] = kk.w;
        in.d[i] = dd.x, in.d[i + 1] = dd.y, in.d[i + 2] = dd.z, in.d[i + 3] = dd.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NPT; ++i) in.q[i] = src[i], in.k[i] = src[NP + i], in.d[i] = src[2 * NP + i];
    }
    in.v = buf[t * ROW + 3 * NP + p];
  };
  // one token: every row of this thread decays and takes its share of k v^T; returns the thread's part of the output
  auto move_rows = [&](const TokenIn& in) __attribute__((always_inline)) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const float kv = in.k[i] * in.v;
      if (BEFORE) {
        acc += (s[i] + u[i] * kv) * in.q[i];
        s[i] = in.d[i] * s[i] + kv;
      } else {
        s[i] = in.d[i] * s[i] + kv;
        acc += s[i] * in.q[i];
      }
    }
    return acc;
  };
  fetch(first);
  put(first, shared);
  shared_memory_barrier();
  int turn = 0;
  for (int c0 = first; c0 < end; c0 += CH) {
    const float* buf = shared + turn * PER_BUF;
    const bool more = c0 + CH < end;
    if (more) fetch(c0 + CH);
    const int n_tok = end - c0 < CH ? end - c0 : CH;
    if constexpr (CH == 1) {
      TokenIn in;
      read_token(buf, 0, in);
      part[r * PC + p] = move_rows(in);
    } else if constexpr (NPT > 4) {
      // many rows a thread: two sets of registers take turns, a token's values are read one token ahead
      const int t_end = (n_tok + 1) & ~1;
      TokenIn in_a, in_b;
      read_token(buf, 0, in_a);
      for (int t = 0; t < t_end; t += 2) {
        read_token(buf, t + 1, in_b);
        part[t * PART + r * PC + p] = move_rows(in_a);
        read_token(buf, t + 2 < CH ? t + 2 : CH - 1, in_a);
        part[(t + 1) * PART + r * PC + p] = move_rows(in_b);
      }
    } else {
      // four sets of registers take turns: a token's values are read three tokens ahead of the arithmetic that uses
      // them, so that the reads' way through shared memory passes behind the work on the tokens before (tokens past
      // the entry's end were staged with k = 0 and a decay of one: they change nothing)
      // (the whole chunk is walked, so that the loop unrolls and every address in shared memory is a constant)
      TokenIn in0, in1, in2, in3;
      auto at = [](int t) __attribute__((always_inline)) { return t < CH ? t : CH - 1; };
      read_token(buf, 0, in0);
      read_token(buf, at(1), in1);
      read_token(buf, at(2), in2);
#pragma unroll
      for (int t = 0; t < CH; t += 4) {
        read_token(buf, at(t + 3), in3);
        part[t * PART + r * PC + p] = move_rows(in0);
        read_token(buf, at(t + 4), in0);
        part[(t + 1) * PART + r * PC + p] = move_rows(in1);
        read_token(buf, at(t + 5), in1);
        part[(t + 2) * PART + r * PC + p] = move_rows(in2);
        read_token(buf, at(t + 6), in2);
        part[(t + 3) * PART + r * PC + p] = move_rows(in3);
      }
    }
    // the next chunk goes to the other buffer before this chunk's results are stored: the wait for its loads then
    // does not also wait for those stores (loads and stores are counted together, in order)
    if (more) put(c0 + CH, shared + (1 - turn) * PER_BUF);
    shared_memory_barrier();
    for (int e = tid; e < n_tok * PC; e += SCAN_THREADS) {
      const int t = e / PC, pp = e % PC;
      if (p0 + pp < P) {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) sum += part[t * PART + i * PC + pp];
        a.out[(size_t)(c0 + t) * a.heads * P + h * P + p0 + pp] = sum;
      }
    }
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

template <int PC, int NPT, bool BEFORE, int CH, bool VEC = false>
static int launch_decay_scan_as(const ScanArgs& a, int B_, hipStream_t stream) {
  constexpr int R = SCAN_THREADS / PC, NP = R * NPT;
  constexpr size_t need = (2 * (size_t)CH * (3 * NP + PC) + (size_t)CH * (R * PC + (PC < 64 ? PC : 0))) * sizeof(float);
  static_assert(need <= 160 * 1024, "a block's staging fits the shared memory of a compute unit");
  if (need > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute((const void*)decay_scan_kernel<PC, NPT, BEFORE, CH, VEC>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)need);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL((decay_scan_kernel<PC, NPT, BEFORE, CH, VEC>), dim3(B_, a.heads, (a.P + PC - 1) / PC), dim3(SCAN_THREADS),
                     need, stream, a);
  ULLM_LAUNCH_CHECK();
}

// 16-byte pieces on the way into shared memory: rows and offsets that are multiples of four values
static bool scan_rows_in_pieces(const ScanArgs& a) {
  const bool raw_decays = a.decay_kind != DECAY_PER_HEAD;       // else z holds the heads' constants and is not staged
  return a.N % 4 == 0 && a.P % 4 == 0 && a.q_ld % 4 == 0 && a.k_ld % 4 == 0 && a.v_ld % 4 == 0 &&
         ((uintptr_t)a.q | (uintptr_t)a.k | (uintptr_t)a.v) % 16 == 0 &&
         (!raw_decays || (a.z_ld % 4 == 0 && (uintptr_t)a.z % 16 == 0));
}

template <int PC, int NPT>
static int launch_decay_scan(const ScanArgs& a, int B_, bool single, hipStream_t stream) {
  // tokens a chunk: 16, or 8 where a slice of 16 has 128 key channels or more to stage (four blocks of a compute unit
  // then fit its shared memory instead of two: 836 -> 663 us for eight prompts of 1024 tokens at 128 x 128 a head)
  constexpr int CHUNK = (PC == 16 && SCAN_THREADS / PC * NPT >= 128) ? SCAN_CHUNK / 2 : SCAN_CHUNK;
  if (single) return a.before ? launch_decay_scan_as<PC, NPT, true, 1>(a, B_, stream)
                              : launch_decay_scan_as<PC, NPT, false, 1>(a, B_, stream);
  if constexpr ((SCAN_THREADS / PC * NPT) % 4 == 0) {
    if (scan_rows_in_pieces(a))
      return a.before ? launch_decay_scan_as<PC, NPT, true, CHUNK, true>(a, B_, stream)
                      : launch_decay_scan_as<PC, NPT, false, CHUNK, true>(a, B_, stream);
  }
  return a.before ? launch_decay_scan_as<PC, NPT, true, CHUNK>(a, B_, stream)
                  : launch_decay_scan_as<PC, NPT, false, CHUNK>(a, B_, stream);
}

// Few blocks: longer chunks (fewer waits for the next chunk's values with nothing else to run meanwhile) and, where
// the rows allow it, 16-byte pieces on their way into shared memory.
template <int PC, int NPT, int CH>
static int launch_decay_scan_few(const ScanArgs& a, int B_, hipStream_t stream) {
  const bool vec = scan_rows_in_pieces(a);
  if (vec) return a.before ? launch_decay_scan_as<PC, NPT, true, CH, true>(a, B_, stream)
                           : launch_decay_scan_as<PC, NPT, false, CH, true>(a, B_, stream);
  return a.before ? launch_decay_scan_as<PC, NPT, true, CH>(a, B_, stream)
                  : launch_decay_scan_as<PC, NPT, false, CH>(a, B_, stream);
}

// max_len: the most tokens any entry brings (1: a step of single tokens).
extern "C" int ullm_decay_scan(const float* q, int q_ld, const float* k, int k_ld, const float* v, int v_ld, const float* z,
                               int z_ld, int decay_kind, float tau, const float* bonus, int silu_inputs, float q_scale,
                               int before, float* state, long long state_stride, long long state_off,
                               const int* q_start, const int* entry_slot, float* out, int B_, int heads, int N, int P,
                               int write_state, int max_len, hipStream_t stream) {
  if (B_ <= 0) return 0;
  if (heads <= 0 || N <= 0 || P <= 0 || N > 512) return ULLM_ERR_SHAPE;
  if (decay_kind < DECAY_PER_HEAD || decay_kind > DECAY_READY || z == nullptr) return ULLM_ERR_UNSUPPORTED;
  if (decay_kind == DECAY_SIGMOID_ROOT && !(tau > 0.f)) return ULLM_ERR_UNSUPPORTED;
  ScanArgs a;
  a.q = q, a.k = k, a.v = v, a.z = z, a.bonus = bonus, a.state = state, a.state_stride = state_stride, a.state_off = state_off;
  a.q_start = q_start, a.entry_slot = entry_slot, a.out = out, a.q_ld = q_ld, a.k_ld = k_ld, a.v_ld = v_ld, a.z_ld = z_ld;
  a.heads = heads, a.N = N, a.P = P, a.decay_kind = decay_kind, a.silu_inputs = silu_inputs, a.before = before;
  a.write_state = write_state, a.q_scale = q_scale, a.inv_tau = decay_kind == DECAY_SIGMOID_ROOT ? 1.f / tau : 1.f;
  const bool single = max_len == 1;
#define SCAN_GO(PC, NPT) return launch_decay_scan<PC, NPT>(a, B_, single, stream)
  // whole rows of 64 value channels a block where there are blocks enough without slicing the heads (a step of
  // many requests: the state's rows then move as whole lines); else slices of 16
  if (P % 64 == 0 && N <= 128 && (long long)B_ * heads >= 1024) {
    if (N <= 32) SCAN_GO(64, 8);
    if (N <= 64) SCAN_GO(64, 16);
    SCAN_GO(64, 32);
  }
  // few blocks (one long prompt): slices of 8, so that twice as many compute units have a block
  if (!single && N <= 256 && (long long)B_ * heads * ((P + 15) / 16) < 256) {
    if (N <= 32) return launch_decay_scan_few<8, 1, 32>(a, B_, stream);
    if (N <= 64) return launch_decay_scan_few<8, 2, 32>(a, B_, stream);
    if (N <= 128) return launch_decay_scan_few<8, 4, 32>(a, B_, stream);
    return launch_decay_scan_few<8, 8, SCAN_CHUNK>(a, B_, stream);
  }
  if (N <= 16) SCAN_GO(16, 1);
  if (N <= 32) SCAN_GO(16, 2);
  if (N <= 64) SCAN_GO(16, 4);
  if (N <= 128) SCAN_GO(16, 8);
  if (N <= 256) SCAN_GO(16, 16);
  SCAN_GO(16, 32);
#undef SCAN_GO
}

// ------------------------------------------------------------------ the inputs' functions, ahead of the recurrence
// For steps of many tokens: silu over a column range of the projection's rows and the decay's function over the raw
// decays, both in place, once per value (the recurrence's blocks, one per slice of value channels, would each apply
// them again).  The same functions as inside the recurrence: a value has the same bits whichever applied them.
__global__ void __launch_bounds__(256)
decay_prepare_kernel(float* __restrict__ x, int x_ld, int x_cols, float* __restrict__ z, int z_ld, int z_cols, int decay_kind,
                     float inv_tau, int T_) {
  const int cols = x_cols + z_cols;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)T_ * cols) return;
  const int t = (int)(i / cols), c = (int)(i % cols);
  if (c < x_cols) {
    float* p = x + (size_t)t * x_ld + c;
    *p = exact_silu(*p);
  } else {
    float* p = z + (size_t)t * z_ld + (c - x_cols);
    *p = decay_of(*p, decay_kind, inv_tau);
  }
}

extern "C" int ullm_decay_prepare(float* x, int x_ld, int x_cols, float* z, int z_ld, int z_cols, int decay_kind, float tau,
                                  int T_, hipStream_t stream) {
  if (T_ <= 0 || x_cols + z_cols <= 0) return 0;
  if (x_cols < 0 || z_cols < 0 || (x_cols && !x) || (z_cols && !z)) return ULLM_ERR_SHAPE;
  if (z_cols && decay_kind != DECAY_SIGMOID_ROOT && decay_kind != DECAY_EXP_EXP) return ULLM_ERR_UNSUPPORTED;
  if (z_cols && decay_kind == DECAY_SIGMOID_ROOT && !(tau > 0.f)) return ULLM_ERR_UNSUPPORTED;
  const size_t n = (size_t)T_ * (x_cols + z_cols);
  hipLaunchKernelGGL(decay_prepare_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, x_ld, x_cols, z, z_ld,
                     z_cols, decay_kind, decay_kind == DECAY_SIGMOID_ROOT ? 1.f / tau : 1.f, T_);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ token shift
// out[m, t, :] = x[t] + (prev(t) - x[t]) * mu[m] for m < M, with prev(t) the row before t in its entry or, for an
// entry's first token, what the state row holds (the last row of the step before; zeros at a request's start).
// The block of an entry's first token then puts the entry's last row into the state row: a thread reads the old
// value of a column before it writes the new one.
// V columns a thread (4 where the rows allow 16-byte pieces, 8-byte ones of bfloat16), as many threads as the row
// has such pieces, up to 1024.
template <typename T, int V>
__global__ void __launch_bounds__(1024)
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
  for (int col = V * threadIdx.x; col < H; col += V * blockDim.x) {
    float cur[V], diff[V], keep[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
      cur[j] = ld_f32(x + (size_t)t * H + col + j);
      const float prev = head ? row[col + j] : ld_f32(x + (size_t)(t - 1) * H + col + j);
      diff[j] = prev - cur[j];
      keep[j] = (head && write_state) ? ld_f32(x + (size_t)last * H + col + j) : 0.f;
    }
    for (int m = 0; m < M; ++m) {
#pragma unroll
      for (int j = 0; j < V; ++j) st_f32(out + ((size_t)m * T_ + t) * H + col + j, cur[j] + diff[j] * mu[(size_t)m * H + col + j]);
    }
    if (head && write_state) {
#pragma unroll
      for (int j = 0; j < V; ++j) row[col + j] = keep[j];
    }
  }
}

extern "C" int ullm_token_shift(const void* x, const float* mu, float* state, long long state_stride, long long state_off,
                                const int* token_entry, const int* q_start, const int* entry_slot, void* out, int T_,
                                int H, int M, int write_state, int dtype, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (H < 1 || M < 1) return ULLM_ERR_SHAPE;
  const bool vec = H % 4 == 0;
  const int pieces = vec ? H / 4 : H;
  int threads = 64;
  while (threads < pieces && threads < 1024) threads *= 2;
#define SHIFT_GO(TT, V) hipLaunchKernelGGL((token_shift_kernel<TT, V>), dim3(T_), dim3(threads), 0, stream, (const TT*)x, mu, state, \
    state_stride, state_off, token_entry, q_start, entry_slot, (TT*)out, T_, H, M, write_state)
  if (dtype == ULLM_F32) { if (vec) SHIFT_GO(float, 4); else SHIFT_GO(float, 1); }
  else if (dtype == ULLM_BF16) { if (vec) SHIFT_GO(bf16_t, 4); else SHIFT_GO(bf16_t, 1); }
  else return ULLM_ERR_DTYPE;
#undef SHIFT_GO
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ norm of the outputs, gain and gate
// The row o [width] is cut into `parts` equal parts (the heads, or one part); each is divided by its root mean
// square (eps inside the root), multiplied by gain[c % gain_len] (a gain per value channel shared by the heads, or
// one per column) and by silu or sigmoid of the gate's raw value g[t, c].  Parts of up to 1024 values: a wave per
// (token, part), every lane's values in registers between the sum of squares and the scaling; longer parts: a block.
#define NORM_PER_LANE 16
// `slices` > 1: o is [slices, T, width] and a value is the sum of its slices, added in their order.
__device__ __forceinline__ float sum_slices(const float* p, int slices, size_t stride) {
  float v = p[0];
  for (int s = 1; s < slices; ++s) v += p[(size_t)s * stride];
  return v;
}

template <typename TO>
__global__ void __launch_bounds__(256)
gated_unit_norm_wave_kernel(const float* __restrict__ o, const float* __restrict__ g, int g_ld, const float* __restrict__ gain,
                            int gain_len, float eps, int gate_kind, TO* __restrict__ out, int T_, int width, int parts,
                            int slices) {
  const int lane = threadIdx.x % WAVE;
  const long long item = (long long)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
  if (item >= (long long)T_ * parts) return;
  const int t = (int)(item / parts), part = (int)(item % parts);
  const int size = width / parts;
  const float* src = o + (size_t)t * width + (size_t)part * size;
  float v[NORM_PER_LANE], z[NORM_PER_LANE];
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NORM_PER_LANE; ++i) {
    const int c = lane + WAVE * i;
    v[i] = c < size ? sum_slices(src + c, slices, (size_t)T_ * width) : 0.f;
    z[i] = c < size ? g[(size_t)t * g_ld + part * size + c] : 0.f;
    sq += v[i] * v[i];
  }
  const float r = 1.f / sqrtf(wave_sum(sq) / (float)size + eps);
#pragma unroll
  for (int i = 0; i < NORM_PER_LANE; ++i) {
    const int c = lane + WAVE * i;
    if (c < size) {
      const int col = part * size + c;
      const float gate = gate_kind == GATE_SIGMOID ? 1.f / (1.f + expf(-z[i])) : exact_silu(z[i]);
      st_f32(out + (size_t)t * width + col, v[i] * r * gain[col % gain_len] * gate);
    }
  }
}

template <typename TO>
__global__ void __launch_bounds__(1024)
gated_unit_norm_block_kernel(const float* __restrict__ o, const float* __restrict__ g, int g_ld, const float* __restrict__ gain,
                             int gain_len, float eps, int gate_kind, TO* __restrict__ out, int T_, int width, int parts,
                             int slices) {
  __shared__ float scratch[16];
  const int t = blockIdx.x / parts, part = blockIdx.x % parts;
  const int size = width / parts;
  const float* src = o + (size_t)t * width + (size_t)part * size;
  const size_t stride = (size_t)T_ * width;
  float sq = 0.f;
  for (int c = threadIdx.x; c < size; c += blockDim.x) {
    const float x = sum_slices(src + c, slices, stride);
    sq += x * x;
  }
  const float r = 1.f / sqrtf(block_sum(sq, scratch) / (float)size + eps);
  for (int c = threadIdx.x; c < size; c += blockDim.x) {
    const int col = part * size + c;
    const float z = g[(size_t)t * g_ld + col];
    const float gate = gate_kind == GATE_SIGMOID ? 1.f / (1.f + expf(-z)) : exact_silu(z);
    st_f32(out + (size_t)t * width + col, sum_slices(src + c, slices, stride) * r * gain[col % gain_len] * gate);
  }
}

extern "C" int ullm_gated_unit_norm(const float* o, const float* g, int g_ld, const float* gain, int gain_len, float eps,
                                    int gate_kind, void* out, int T_, int width, int parts, int slices, int out_dtype,
                                    hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (width < 1 || parts < 1 || width % parts || gain_len < 1 || width % gain_len || slices < 1) return ULLM_ERR_SHAPE;
  if (gate_kind != GATE_SILU && gate_kind != GATE_SIGMOID) return ULLM_ERR_UNSUPPORTED;
  if (out_dtype != ULLM_F32 && out_dtype != ULLM_BF16) return ULLM_ERR_DTYPE;
  const int size = width / parts;
  if (size <= WAVE * NORM_PER_LANE) {
    const long long items = (long long)T_ * parts;
    const dim3 grid((unsigned)((items + 3) / 4));
    if (out_dtype == ULLM_F32)
      hipLaunchKernelGGL(gated_unit_norm_wave_kernel<float>, grid, dim3(256), 0, stream, o, g, g_ld, gain, gain_len, eps,
                         gate_kind, (float*)out, T_, width, parts, slices);
    else
      hipLaunchKernelGGL(gated_unit_norm_wave_kernel<bf16_t>, grid, dim3(256), 0, stream, o, g, g_ld, gain, gain_len, eps,
                         gate_kind, (bf16_t*)out, T_, width, parts, slices);
  } else {
    int threads = 256;
    while (threads < size / 4 && threads < 1024) threads *= 2;
    const dim3 grid((unsigned)((long long)T_ * parts));
    if (out_dtype == ULLM_F32)
      hipLaunchKernelGGL(gated_unit_norm_block_kernel<float>, grid, dim3(threads), 0, stream, o, g, g_ld, gain, gain_len, eps,
                         gate_kind, (float*)out, T_, width, parts, slices);
    else
      hipLaunchKernelGGL(gated_unit_norm_block_kernel<bf16_t>, grid, dim3(threads), 0, stream, o, g, g_ld, gain, gain_len, eps,
                         gate_kind, (bf16_t*)out, T_, width, parts, slices);
  }
  ULLM_LAUNCH_CHECK();
}
