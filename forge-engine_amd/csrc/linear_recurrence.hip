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
// Work split: block = (8 value columns, head, sequence), 128 threads.  Thread (rg = tid % 16,
// jl = tid / 16) owns column jl of the block and the R key channels rg * R .. rg * R + R - 1 of that
// column's state in registers for the whole walk; the 16 lanes of a column meet by lane permutes.
// Tokens are staged a chunk (16, or 8 for key sizes beyond 128) at a time through LDS: q, k, the
// decay per key channel with its transform applied, v times the input scale, the per-head decay.
// The exponentials of the decays are thus computed by all threads at once and the walk itself is
// multiply-adds.  The next chunk's loads are issued into registers before the walk over this
// chunk begins, so that memory latency hides behind the walk.  A block's columns are its own, so
// nothing is shared between blocks and the state is read once and written once per step.
// Decays: per key channel, kind 1  a = exp(-exp(d + bias)),  kind 2  a = sigmoid(d + bias)^(1 / tau)
// = exp(logsigmoid(d + bias) / tau); or one factor per head and token (not both).  One more
// column fed by v = 1 (`ones_column`) follows the recurrence with k alone: a normaliser.
#include "common.h"

#define LR_THREADS 128
#define LR_COLS 8

__device__ __forceinline__ float sum_16_lanes(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // lane ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // 7 - lane within 8
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // 15 - lane within 16
  return v;
}

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

__device__ __forceinline__ float load_either(const void* p, size_t index, bool is_bf16) {
  return is_bf16 ? bf16_to_float(((const bf16_t*)p)[index]) : ((const float*)p)[index];
}

struct RecurrenceArgs {
  const void* q; const void* k; const void* v;
  size_t q_stride, k_stride, v_stride;
  const float* decay; const float* decay_bias; const float* head_decay; const float* in_scale; const float* bonus;
  float* state; float* out;
  const int* cu_q; const int* state_slots;
  float tau, q_scale;
  int is_bf16, decay_kind, ones_column, slots, heads, key_dim, value_dim, tokens;
};

// CHANNEL: the decay comes per key channel (p.decay with its transform); else per head and token
// (p.head_decay, or none at all: 1).
template <int R, bool BONUS, bool CHANNEL>
__global__ __launch_bounds__(LR_THREADS) void linear_recurrence_kernel(RecurrenceArgs p) {
  constexpr int DKP = 16 * R;                  // key channels, padded
  constexpr int CH = R > 8 ? 8 : 16;           // tokens a chunk
  constexpr int E = CH * DKP / LR_THREADS;     // elements of a chunk's q (and k, and decay) a thread stages
  __shared__ float Qs[CH][DKP];
  __shared__ float Ks[CH][DKP];
  __shared__ float As[CHANNEL ? CH : 1][DKP];
  __shared__ float Vs[CH][LR_COLS];
  __shared__ float Hd[CH];
  __shared__ float Bs[DKP];

  const int seq = blockIdx.z, h = blockIdx.y, j0 = blockIdx.x * LR_COLS;
  const int begin = p.cu_q[seq], end = p.cu_q[seq + 1];
  const int slot = p.state_slots[seq];
  if (end <= begin || end > p.tokens || slot < 0 || slot >= p.slots) return;
  const int tid = threadIdx.x, rg = tid & 15, jl = tid >> 4;
  const int Dk = p.key_dim, Dv = p.value_dim, H = p.heads;
  const int columns = Dv + p.ones_column;
  const int col = j0 + jl;
  const bool is_bf16 = p.is_bf16 != 0;

  float S[R], U[R];
  float* mine = p.state + (((size_t)slot * H + h) * columns + min(col, columns - 1)) * Dk;
#pragma unroll
  for (int m = 0; m < R; ++m) {
    const int i = rg * R + m;
    S[m] = (col < columns && i < Dk) ? mine[i] : 0.f;
    U[m] = (BONUS && i < Dk) ? p.bonus[(size_t)h * Dk + i] : 0.f;
  }
  if (CHANNEL)
    for (int i = tid; i < DKP; i += LR_THREADS) Bs[i] = i < Dk ? p.decay_bias[(size_t)h * Dk + i] : 0.f;

  // a chunk's loads, into registers: every load is unconditional (indices past the end are clamped, what
  // they bring is dropped when the chunk is staged)
  float qr[E], kr[E], dr[CHANNEL ? E : 1], vr = 0.f, sr = 1.f, hr = 1.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int n = 0; n < E; ++n) {
      const int e = tid + n * LR_THREADS;
      const int tt = e / DKP, i = e - tt * DKP;
      const size_t t = (size_t)min(t0 + tt, end - 1);
      const size_t c = (size_t)h * Dk + min(i, Dk - 1);
      qr[n] = load_either(p.q, t * p.q_stride + c, is_bf16);
      kr[n] = load_either(p.k, t * p.k_stride + c, is_bf16);
      if (CHANNEL) dr[n] = p.decay[t * H * Dk + c];
    }
    if (tid < CH * LR_COLS) {
      const int tt = tid / LR_COLS, c = j0 + tid % LR_COLS;
      const size_t t = (size_t)min(t0 + tt, end - 1);
      vr = load_either(p.v, t * p.v_stride + (size_t)h * Dv + min(c, Dv - 1), is_bf16);
      if (c >= Dv) vr = c < columns ? 1.f : 0.f;
      sr = p.in_scale ? p.in_scale[t * H + h] : 1.f;
    }
    if (tid < CH) hr = p.head_decay ? p.head_decay[(size_t)min(t0 + tid, end - 1) * H + h] : 1.f;
  };
  auto stage = [&](int t0) {
#pragma unroll
    for (int n = 0; n < E; ++n) {
      const int e = tid + n * LR_THREADS;
      const int tt = e / DKP, i = e - tt * DKP;
      const bool live = t0 + tt < end && i < Dk;
      Qs[tt][i] = live ? qr[n] * p.q_scale : 0.f;
      Ks[tt][i] = live ? kr[n] : 0.f;
      if (CHANNEL) {
        const float z = dr[n] + Bs[i];
        const float a = p.decay_kind == 1 ? expf(-expf(z)) : expf(log_sigmoid(z) / p.tau);
        As[tt][i] = live ? a : 1.f;
      }
    }
    if (tid < CH * LR_COLS) Vs[tid / LR_COLS][tid % LR_COLS] = t0 + tid / LR_COLS < end ? vr * sr : 0.f;
    if (tid < CH) Hd[tid] = hr;
  };

  fetch(begin);
  for (int t0 = begin; t0 < end; t0 += CH) {
    __syncthreads();     // the chunk before is consumed (and the bias row is in place)
    stage(t0);
    __syncthreads();
    if (t0 + CH < end) fetch(t0 + CH);      // in flight while this chunk is walked

    const int count = min(CH, end - t0);
    for (int tt = 0; tt < count; ++tt) {
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
      acc = sum_16_lanes(acc);
      if (rg == 0 && col < columns) p.out[((size_t)(t0 + tt) * H + h) * columns + col] = acc;
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

template <int R>
static void launch_recurrence(const RecurrenceArgs& p, dim3 grid, hipStream_t stream) {
  if (p.bonus && p.decay_kind) linear_recurrence_kernel<R, true, true><<<grid, LR_THREADS, 0, stream>>>(p);
  else if (p.bonus) linear_recurrence_kernel<R, true, false><<<grid, LR_THREADS, 0, stream>>>(p);
  else if (p.decay_kind) linear_recurrence_kernel<R, false, true><<<grid, LR_THREADS, 0, stream>>>(p);
  else linear_recurrence_kernel<R, false, false><<<grid, LR_THREADS, 0, stream>>>(p);
}

extern "C" int fe_linear_recurrence(const void* q, const void* k, const void* v, int dtype, long long q_stride,
                                    long long k_stride, long long v_stride, const float* decay, int decay_kind,
                                    const float* decay_bias, float tau, const float* head_decay, const float* in_scale,
                                    float q_scale, const float* bonus, int ones_column, float* state, int slots,
                                    float* out, const int* cu_q, const int* state_slots, int num_seqs, int max_q_len,
                                    int heads, int key_dim, int value_dim, int tokens, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (heads <= 0 || key_dim < 1 || key_dim > 256 || value_dim < 1 || slots < 1 || max_q_len < 1 ||
      (dtype != FE_F32 && dtype != FE_BF16) || decay_kind < 0 || decay_kind > 2 || (decay_kind && (!decay || !decay_bias)) ||
      !(tau > 0.f) || heads > 65535 || num_seqs > 65535 || (decay_kind && head_decay))
    return FE_BAD_ARGUMENT;
  if (q_stride < (long long)heads * key_dim || k_stride < (long long)heads * key_dim || v_stride < (long long)heads * value_dim)
    return FE_BAD_ARGUMENT;
  RecurrenceArgs p;
  p.q = q; p.k = k; p.v = v;
  p.q_stride = (size_t)q_stride; p.k_stride = (size_t)k_stride; p.v_stride = (size_t)v_stride;
  p.decay = decay; p.decay_bias = decay_bias; p.head_decay = head_decay; p.in_scale = in_scale; p.bonus = bonus;
  p.state = state; p.out = out; p.cu_q = cu_q; p.state_slots = state_slots;
  p.tau = tau; p.q_scale = q_scale;
  p.is_bf16 = dtype == FE_BF16; p.decay_kind = decay_kind; p.ones_column = ones_column ? 1 : 0; p.slots = slots;
  p.heads = heads; p.key_dim = key_dim; p.value_dim = value_dim; p.tokens = tokens;
  const int columns = value_dim + p.ones_column;
  const dim3 grid((columns + LR_COLS - 1) / LR_COLS, heads, num_seqs);
  const int r = (key_dim + 15) / 16;
  if (r <= 1) launch_recurrence<1>(p, grid, stream);
  else if (r <= 2) launch_recurrence<2>(p, grid, stream);
  else if (r <= 3) launch_recurrence<3>(p, grid, stream);
  else if (r <= 4) launch_recurrence<4>(p, grid, stream);
  else if (r <= 6) launch_recurrence<6>(p, grid, stream);
  else if (r <= 8) launch_recurrence<8>(p, grid, stream);
  else if (r <= 12) launch_recurrence<12>(p, grid, stream);
  else launch_recurrence<16>(p, grid, stream);
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
