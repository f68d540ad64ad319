// Linear recurrences over a matrix state, for mixers that carry a state instead of a cache of keys
// (RWKV time mixing, gated linear attention, the matrix memory of xLSTM).  Per sequence and head,
// token after token:
//     S <- diag(a_t) S + b_t k_t v_t^T          S: [key dim][value dim], float32
//     o_t = S^T q_t                              (read after the update), or
//     o_t = (S_before + diag(u) b_t k_t v_t^T)^T q_t   (read before it, with a bonus u for the token itself)
// The state of every live request lives in a slot of `state` [slots][heads][columns][key dim]
// (value-major) and is carried from step to step, so a request may be cut into steps anywhere; a
// step may hold portions of prompts beside single tokens.
//
// Work split: block = 256 threads that share a head's staged tokens; a column of the state belongs to
// L lanes (16 for key sizes up to 64, a whole wave of 64 beyond), each holding R key channels of it
// in registers for the whole walk, so a block owns 16 or 4 columns and the lanes of a column meet by
// lane permutes.  Tokens are staged 16 at a time through LDS (q, k, the decay per key channel, v
// times the input scale, the per-head decay); the next chunk's loads are issued into registers
// before the walk over this chunk begins, every one of them unconditional (a load under a branch
// is waited for at the branch's join, which would serialise them), so that memory latency hides
// behind the walk.  A whole chunk's walk is unrolled: the LDS reads of later tokens overlap the
// sums of earlier ones, and a chunk's results leave in one store per lane.  A block's columns are
// its own, so nothing is shared between blocks and the state is read once and written once per step.
// Decays per key channel arrive ready (a kernel of its own applies their transform to the whole
// step at once: kind 1  a = exp(-exp(d + bias)),  kind 2  a = sigmoid(d + bias)^(1 / tau) =
// exp(logsigmoid(d + bias) / tau)), or there is one factor per head and token (not both).  One more
// column fed by v = 1 (`ones_column`) follows the recurrence with k alone: a normaliser.
#include "common.h"

#define LR_THREADS 256
#define LR_CHUNK 16

__device__ __forceinline__ float sum_16_lanes(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // lane ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // 7 - lane within 8
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // 15 - lane within 16
  return v;
}

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// The element type is a template parameter of the kernel: a choice at run time would put every load
// under a branch, and the wait behind each branch's join would serialise a chunk's loads.
template <bool IS_BF16>
__device__ __forceinline__ float load_either(const void* p, size_t index) {
  return IS_BF16 ? bf16_to_float(((const bf16_t*)p)[index]) : ((const float*)p)[index];
}

__device__ const float lr_one[1] = {1.f};     // what an absent per-head factor reads: loads stay unconditional

struct RecurrenceArgs {
  const void* q; const void* k; const void* v;
  size_t q_stride, k_stride, v_stride;
  const float* decay; const float* head_decay; const float* in_scale; const float* bonus;
  float* state; float* out;
  const int* cu_q; const int* state_slots;
  float q_scale;
  int is_bf16, ones_column, slots, heads, key_dim, value_dim, tokens;
};

// a = exp(-exp(d + bias)) (kind 1) or sigmoid(d + bias)^(1 / tau) (kind 2), in place, for a step's
// decays [rows][width]
__global__ void decay_transform_kernel(float* __restrict__ decay, const float* __restrict__ bias, int kind, float tau,
                                       long long count, int width) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const float z = decay[i] + bias[i % width];
  decay[i] = kind == 1 ? expf(-expf(z)) : expf(log_sigmoid(z) / tau);
}

// L lanes a column, R key channels a lane; CHANNEL: the decay comes per key channel (p.decay, ready),
// else per head and token (p.head_decay, or none at all: 1).
template <int L, int R, bool BONUS, bool CHANNEL, bool IS_BF16>
__global__ __launch_bounds__(LR_THREADS) void linear_recurrence_kernel(RecurrenceArgs p) {
  constexpr int DKP = L * R;                   // key channels, padded
  constexpr int CH = LR_CHUNK;                 // tokens a chunk
  constexpr int COLS = LR_THREADS / L;         // columns a block
  constexpr int E = CH * DKP / LR_THREADS;     // elements of a chunk's q (and k, and decay) a thread stages
  __shared__ float Qs[CH][DKP];
  __shared__ float Ks[CH][DKP];
  __shared__ float As[CHANNEL ? CH : 1][DKP];
  __shared__ float Vs[CH][COLS];
  __shared__ float Hd[CH];

  const int seq = blockIdx.z, h = blockIdx.y, j0 = blockIdx.x * COLS;
  const int begin = p.cu_q[seq], end = p.cu_q[seq + 1];
  const int slot = p.state_slots[seq];
  if (end <= begin || end > p.tokens || slot < 0 || slot >= p.slots) return;
  const int tid = threadIdx.x, rg = tid % L, jl = tid / L;
  const int Dk = p.key_dim, Dv = p.value_dim, H = p.heads;
  const int columns = Dv + p.ones_column;
  const int col = j0 + jl;

  float S[R], U[R];
  float* mine = p.state + (((size_t)slot * H + h) * columns + min(col, columns - 1)) * Dk;
#pragma unroll
  for (int m = 0; m < R; ++m) {
    const int i = rg * R + m;
    S[m] = (col < columns && i < Dk) ? mine[i] : 0.f;
    U[m] = (BONUS && i < Dk) ? p.bonus[(size_t)h * Dk + i] : 0.f;
  }

  // a chunk's loads, into registers: every load is unconditional (indices past the end are clamped, what
  // they bring is dropped when the chunk is staged)
  float qr[E], kr[E], dr[CHANNEL ? E : 1], vr = 0.f, sr = 1.f, hr = 1.f;
  const float* scale_from = p.in_scale ? p.in_scale : lr_one;
  const float* decay_from = p.head_decay ? p.head_decay : lr_one;
  const size_t scale_step = p.in_scale ? 1 : 0, decay_step = p.head_decay ? 1 : 0;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int n = 0; n < E; ++n) {
      const int e = tid + n * LR_THREADS;
      const int tt = e / DKP, i = e - tt * DKP;
      const size_t t = (size_t)min(t0 + tt, end - 1);
      const size_t c = (size_t)h * Dk + min(i, Dk - 1);
      qr[n] = load_either<IS_BF16>(p.q, t * p.q_stride + c);
      kr[n] = load_either<IS_BF16>(p.k, t * p.k_stride + c);
      if (CHANNEL) dr[n] = p.decay[t * H * Dk + c];
    }
    {   // every thread loads (threads beyond the chunk's values repeat others'): no load under a condition
      const int u = tid % (CH * COLS);
      const int tt = u / COLS, c = j0 + u % COLS;
      const size_t t = (size_t)min(t0 + tt, end - 1);
      vr = load_either<IS_BF16>(p.v, t * p.v_stride + (size_t)h * Dv + min(c, Dv - 1));
      vr = c >= Dv ? (c < columns ? 1.f : 0.f) : vr;
      sr = scale_from[(t * H + h) * scale_step];
      hr = decay_from[((size_t)min(t0 + tid % CH, end - 1) * H + h) * decay_step];
    }
  };
  auto stage = [&](int t0) {
#pragma unroll
    for (int n = 0; n < E; ++n) {
      const int e = tid + n * LR_THREADS;
      const int tt = e / DKP, i = e - tt * DKP;
      const bool live = t0 + tt < end && i < Dk;
      Qs[tt][i] = live ? qr[n] * p.q_scale : 0.f;
      Ks[tt][i] = live ? kr[n] : 0.f;
      if (CHANNEL) As[tt][i] = live ? dr[n] : 1.f;
    }
    if (tid < CH * COLS) Vs[tid / COLS][tid % COLS] = t0 + tid / COLS < end ? vr * sr : 0.f;
    if (tid < CH) Hd[tid] = hr;
  };

  fetch(begin);
  for (int t0 = begin; t0 < end; t0 += CH) {
    __syncthreads();     // the chunk before is consumed
    stage(t0);
    __syncthreads();
    fetch(t0 + CH);      // in flight while this chunk is walked (unconditional: past the end the indices are clamped)

    // one token: the state's update and the read-out, summed over the column's lanes (every lane gets the sum)
    auto token = [&](int tt) -> float {
      const float vj = Vs[tt][jl];
      const float hd = CHANNEL ? 1.f : Hd[tt];
      float acc = 0.f;
#pragma unroll
      for (int m = 0; m < R; ++m) {
        const int i = rg * R + m;
        const float kv = Ks[tt][i] * vj;
        const float a = CHANNEL ? As[tt][i] : hd;
        if (BONUS) {
          acc = fmaf(fmaf(U[m], kv, S[m]), Qs[tt][i], acc);
          S[m] = fmaf(S[m], a, kv);
        } else {
          S[m] = fmaf(S[m], a, kv);
          acc = fmaf(S[m], Qs[tt][i], acc);
        }
      }
      return L == 16 ? sum_16_lanes(acc) : wave_sum_dpp(acc);
    };
    const int count = min(CH, end - t0);
    if (count == CH) {      // a whole chunk, unrolled: the LDS reads of later tokens overlap the sums of earlier ones
      float mine_out = 0.f;
#pragma unroll
      for (int tt = 0; tt < CH; ++tt) {
        const float o = token(tt);
        mine_out = rg == tt ? o : mine_out;     // lane tt of the column keeps token tt's result
      }
      if (rg < CH && col < columns) p.out[((size_t)(t0 + rg) * H + h) * columns + col] = mine_out;
    } else {
      for (int tt = 0; tt < count; ++tt) {
        const float o = token(tt);
        if (rg == 0 && col < columns) p.out[((size_t)(t0 + tt) * H + h) * columns + col] = o;
      }
    }
  }

  if (col < columns) {
#pragma unroll
    for (int m = 0; m < R; ++m) {
      const int i = rg * R + m;
      if (i < Dk) mine[i] = S[m];
    }
  }
}

template <int L, int R, bool IS_BF16>
static void launch_typed(const RecurrenceArgs& p, dim3 grid, hipStream_t stream) {
  if (p.bonus && p.decay) linear_recurrence_kernel<L, R, true, true, IS_BF16><<<grid, LR_THREADS, 0, stream>>>(p);
  else if (p.bonus) linear_recurrence_kernel<L, R, true, false, IS_BF16><<<grid, LR_THREADS, 0, stream>>>(p);
  else if (p.decay) linear_recurrence_kernel<L, R, false, true, IS_BF16><<<grid, LR_THREADS, 0, stream>>>(p);
  else linear_recurrence_kernel<L, R, false, false, IS_BF16><<<grid, LR_THREADS, 0, stream>>>(p);
}

template <int L, int R>
static void launch_recurrence(const RecurrenceArgs& p, int columns, int num_seqs, hipStream_t stream) {
  const dim3 grid((columns + LR_THREADS / L - 1) / (LR_THREADS / L), p.heads, num_seqs);
  if (p.is_bf16) launch_typed<L, R, true>(p, grid, stream);
  else launch_typed<L, R, false>(p, grid, stream);
}

// `decay` (float32 [tokens][heads * key_dim], or null) is transformed IN PLACE first when decay_kind is 1 or
// 2 (see the top of the file); decay_kind 0 with a decay: the values are ready.
extern "C" int fe_linear_recurrence(const void* q, const void* k, const void* v, int dtype, long long q_stride,
                                    long long k_stride, long long v_stride, float* decay, int decay_kind,
                                    const float* decay_bias, float tau, const float* head_decay, const float* in_scale,
                                    float q_scale, const float* bonus, int ones_column, float* state, int slots,
                                    float* out, const int* cu_q, const int* state_slots, int num_seqs, int max_q_len,
                                    int heads, int key_dim, int value_dim, int tokens, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (heads <= 0 || key_dim < 1 || key_dim > 256 || value_dim < 1 || slots < 1 || max_q_len < 1 ||
      (dtype != FE_F32 && dtype != FE_BF16) || decay_kind < 0 || decay_kind > 2 || (decay_kind && (!decay || !decay_bias)) ||
      !(tau > 0.f) || heads > 65535 || num_seqs > 65535 || (decay && head_decay))
    return FE_BAD_ARGUMENT;
  if (q_stride < (long long)heads * key_dim || k_stride < (long long)heads * key_dim || v_stride < (long long)heads * value_dim)
    return FE_BAD_ARGUMENT;
  if (decay_kind) {
    const long long count = (long long)tokens * heads * key_dim;
    decay_transform_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(decay, decay_bias, decay_kind, tau, count,
                                                                                heads * key_dim);
    if (fe_check_launch() != FE_OK) return FE_LAUNCH_FAILED;
  }
  RecurrenceArgs p;
  p.q = q; p.k = k; p.v = v;
  p.q_stride = (size_t)q_stride; p.k_stride = (size_t)k_stride; p.v_stride = (size_t)v_stride;
  p.decay = decay; p.head_decay = head_decay; p.in_scale = in_scale; p.bonus = bonus;
  p.state = state; p.out = out; p.cu_q = cu_q; p.state_slots = state_slots;
  p.q_scale = q_scale;
  p.is_bf16 = dtype == FE_BF16; p.ones_column = ones_column ? 1 : 0; p.slots = slots;
  p.heads = heads; p.key_dim = key_dim; p.value_dim = value_dim; p.tokens = tokens;
  const int columns = value_dim + p.ones_column;
  if (key_dim <= 16) launch_recurrence<16, 1>(p, columns, num_seqs, stream);
  else if (key_dim <= 32) launch_recurrence<16, 2>(p, columns, num_seqs, stream);
  else if (key_dim <= 48) launch_recurrence<16, 3>(p, columns, num_seqs, stream);
  else if (key_dim <= 64) launch_recurrence<16, 4>(p, columns, num_seqs, stream);
  else if (key_dim <= 128) launch_recurrence<64, 2>(p, columns, num_seqs, stream);
  else if (key_dim <= 192) launch_recurrence<64, 3>(p, columns, num_seqs, stream);
  else launch_recurrence<64, 4>(p, columns, num_seqs, stream);
  return fe_check_launch();
}

// ---------------------------------------------------------------- stabilised gates of an mLSTM
// Per sequence and head, along the tokens:  i = cap tanh((g_i + b_i) / cap),
// f = logsigmoid(cap tanh((g_f + b_f) / cap)),  m_t = max(f + m_(t-1), i);
// out[0] = exp(f + m_(t-1) - m_t), out[1] = exp(i - m_t), out[2] = exp(-m_t).
// One wave per (sequence, head), 64 tokens at a time: the running maximum is a scan over the maps
// m -> max(m + a, b), which compose as (a1, b1) then (a2, b2) = (a1 + a2, max(b1 + a2, b2)).
__global__ __launch_bounds__(64) void mlstm_gate_scan_kernel(const float* __restrict__ gates, const float* __restrict__ bias,
                                                             float cap, float* __restrict__ maximum, int slots,
                                                             const int* __restrict__ cu_q, const int* __restrict__ state_slots,
                                                             float* __restrict__ out, int tokens, int heads) {
  const int seq = blockIdx.y, h = blockIdx.x, lane = threadIdx.x;
  const int begin = cu_q[seq], end = cu_q[seq + 1];
  const int slot = state_slots[seq];
  if (end <= begin || end > tokens || slot < 0 || slot >= slots) return;
  float m_in = maximum[(size_t)slot * heads + h];
  const float bi = bias[h], bf = bias[heads + h];
  const size_t plane = (size_t)tokens * heads;
  for (int t0 = begin; t0 < end; t0 += 64) {
    const int t = t0 + lane;
    const bool live = t < end;
    float gi = -INFINITY, gf = 0.f;     // the identity map for lanes past the end
    if (live) {
      gi = cap * tanhf((gates[(size_t)t * 2 * heads + h] + bi) / cap);
      gf = log_sigmoid(cap * tanhf((gates[(size_t)t * 2 * heads + heads + h] + bf) / cap));
    }
    float a = gf, b = gi;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
      const float pa = __shfl_up(a, offset, 64), pb = __shfl_up(b, offset, 64);
      if (lane >= offset) {
        b = fmaxf(pb + a, b);
        a = pa + a;
      }
    }
    const float m = fmaxf(m_in + a, b);
    float m_before = __shfl_up(m, 1, 64);
    if (lane == 0) m_before = m_in;
    if (live) {
      const size_t at = (size_t)t * heads + h;
      out[at] = expf(gf + m_before - m);
      out[plane + at] = expf(gi - m);
      out[2 * plane + at] = expf(-m);
    }
    m_in = __shfl(m, 63, 64);
  }
  if (lane == 0) maximum[(size_t)slot * heads + h] = m_in;
}

extern "C" int fe_mlstm_gate_scan(const float* gates, const float* bias, float cap, float* maximum, int slots,
                                  const int* cu_q, const int* state_slots, float* out, int tokens, int num_seqs,
                                  int heads, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (heads <= 0 || slots < 1 || !(cap > 0.f) || num_seqs > 65535) return FE_BAD_ARGUMENT;
  mlstm_gate_scan_kernel<<<dim3(heads, num_seqs), 64, 0, stream>>>(gates, bias, cap, maximum, slots, cu_q, state_slots,
                                                                    out, tokens, heads);
  return fe_check_launch();
}
