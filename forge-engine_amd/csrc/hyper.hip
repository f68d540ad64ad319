// Residual streams kept several at a time, the norm that reads them, and two small row kernels.
//
// fe_hyper_norm: one block per row.  With S streams x_0 .. x_(S-1) of a token (S = 1: the plain
// residual stream) and a pending update y (float32, maybe in parts that are added up in order):
//   x_t <- sum_s mix[s][t] x_s + share[t] y      (mix absent: the identity; share absent: ones)
//   u    = sum_t read[t] x_t                      (read absent: ones, the plain sum)
//   out  = (u - mean) / sqrt(var + eps) * w + b   (layer norm; RMS norm: no mean, no bias)
// all in float32 with one rounding at the store.  The new streams are written back unless the call
// serves chosen rows only.  Without `out` the kernel only applies the update.
//
// fe_embed_token_pairs: a token's row of the embedding table plus a row of a second table chosen
// by the token and the one before it; fe_scale_rows: a factor on every element.
#include "common.h"

#define MAX_STREAMS 8

template <typename TO, int S, int VEC, int THREADS>
__global__ __launch_bounds__(THREADS) void hyper_norm_kernel(
    float* __restrict__ streams, long long stream_stride, const float* __restrict__ update, int parts,
    long long part_stride, const float* __restrict__ mix, const float* __restrict__ share,
    const float* __restrict__ read, const float* __restrict__ weight, const float* __restrict__ bias, float eps,
    int rms, TO* __restrict__ out, const int* __restrict__ rows, int W, int store) {
  extern __shared__ float u_row[];      // the row of u, W floats
  __shared__ float scratch[16];
  const int tid = threadIdx.x;
  const long long row = rows ? rows[blockIdx.x] : blockIdx.x;
  float m[S][S], sh[S], rd[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    sh[s] = share ? share[s] : 1.f;
    rd[s] = read ? read[s] : 1.f;
#pragma unroll
    for (int t = 0; t < S; ++t) m[s][t] = mix ? mix[s * S + t] : (s == t ? 1.f : 0.f);
  }
  float total = 0.f;
  for (int c = tid * VEC; c < W; c += THREADS * VEC) {
    float x[S][VEC], y[VEC];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const float* p = streams + s * stream_stride + row * W + c;
      if constexpr (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        x[s][0] = v.x; x[s][1] = v.y; x[s][2] = v.z; x[s][3] = v.w;
      } else {
        x[s][0] = *p;
      }
    }
    if (update) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) y[i] = 0.f;
      for (int part = 0; part < parts; ++part) {
        const float* p = update + part * part_stride + row * W + c;
        if constexpr (VEC == 4) {
          const float4 v = *reinterpret_cast<const float4*>(p);
          y[0] += v.x; y[1] += v.y; y[2] += v.z; y[3] += v.w;
        } else {
          y[0] += *p;
        }
      }
      float fresh[S][VEC];
#pragma unroll
      for (int t = 0; t < S; ++t)
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < S; ++s) acc = fmaf(m[s][t], x[s][i], acc);
          fresh[t][i] = fmaf(sh[t], y[i], acc);
        }
#pragma unroll
      for (int t = 0; t < S; ++t) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) x[t][i] = fresh[t][i];
        if (store) {
          float* p = streams + t * stream_stride + row * W + c;
          if constexpr (VEC == 4) *reinterpret_cast<float4*>(p) = make_float4(x[t][0], x[t][1], x[t][2], x[t][3]);
          else *p = x[t][0];
        }
      }
    }
    if (out) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float u = 0.f;
#pragma unroll
        for (int t = 0; t < S; ++t) u = fmaf(rd[t], x[t][i], u);
        u_row[c + i] = u;
        total += u;
      }
    }
  }
  if (!out) return;
  // a thread reads back only what it wrote itself: no barrier is needed before the passes below
  const float mean = rms ? 0.f : block_sum<true>(total, scratch) / (float)W;
  float squares = 0.f;
  for (int c = tid * VEC; c < W; c += THREADS * VEC)
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float d = u_row[c + i] - mean;
      squares = fmaf(d, d, squares);
    }
  const float variance = block_sum(squares, scratch) / (float)W;
  const float inv = 1.f / sqrtf(variance + eps);
  TO* orow = out + (size_t)blockIdx.x * W;
  for (int c = tid * VEC; c < W; c += THREADS * VEC)
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float v = (u_row[c + i] - mean) * inv * weight[c + i];
      if (bias) v += bias[c + i];
      store_from_float(orow + c + i, v);
    }
}

template <typename TO, int S>
static void launch_hyper(float* streams, long long stream_stride, const float* update, int parts, long long part_stride,
                         const float* mix, const float* share, const float* read, const float* weight,
                         const float* bias, float eps, int rms, void* out, const int* rows, int n_rows, int W, int store,
                         hipStream_t stream) {
  const size_t lds = out ? (size_t)W * sizeof(float) : 0;
  const bool vec = W % 4 == 0 && ((uintptr_t)streams % 16 == 0) && stream_stride % 4 == 0 &&
                   (!update || ((uintptr_t)update % 16 == 0 && part_stride % 4 == 0));
  // a step of few rows is a matter of round trips, not of bytes: more threads a row then (one round of loads a thread)
  if (vec && n_rows <= 512 && W >= 2048)
    hyper_norm_kernel<TO, S, 4, 1024><<<n_rows, 1024, lds, stream>>>(streams, stream_stride, update, parts, part_stride, mix,
                                                                     share, read, weight, bias, eps, rms, (TO*)out, rows, W, store);
  else if (vec)
    hyper_norm_kernel<TO, S, 4, 256><<<n_rows, 256, lds, stream>>>(streams, stream_stride, update, parts, part_stride, mix, share,
                                                                   read, weight, bias, eps, rms, (TO*)out, rows, W, store);
  else
    hyper_norm_kernel<TO, S, 1, 256><<<n_rows, 256, lds, stream>>>(streams, stream_stride, update, parts, part_stride, mix, share,
                                                                   read, weight, bias, eps, rms, (TO*)out, rows, W, store);
}

template <typename TO>
static int dispatch_hyper(int S, float* streams, long long stream_stride, const float* update, int parts,
                          long long part_stride, const float* mix, const float* share, const float* read,
                          const float* weight, const float* bias, float eps, int rms, void* out, const int* rows,
                          int n_rows, int W, int store, hipStream_t stream) {
#define CASE(N)                                                                                                       \
  case N:                                                                                                             \
    launch_hyper<TO, N>(streams, stream_stride, update, parts, part_stride, mix, share, read, weight, bias, eps, rms, \
                        out, rows, n_rows, W, store, stream);                                                         \
    break;
  switch (S) {
    CASE(1) CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8)
    default: return FE_BAD_ARGUMENT;
  }
#undef CASE
  return fe_check_launch();
}

extern "C" int fe_hyper_norm(float* streams, long long stream_stride, int num_streams, const float* update, int parts,
                             long long part_stride, const float* mix, const float* share, const float* read,
                             const float* weight, const float* bias, float eps, int rms, void* out, int out_dtype,
                             const int* rows, int n_rows, int width, int store, hipStream_t stream) {
  if (n_rows <= 0) return FE_OK;
  if (!streams || width <= 0 || width > 16384 || num_streams < 1 || num_streams > MAX_STREAMS || parts < 0 ||
      (update && parts < 1) || (out && !weight) || (!out && !update))
    return FE_BAD_ARGUMENT;
  if (!out || out_dtype == FE_F32)
    return dispatch_hyper<float>(num_streams, streams, stream_stride, update, parts, part_stride, mix, share, read, weight,
                                 bias, eps, rms, out, rows, n_rows, width, store, stream);
  if (out_dtype == FE_BF16)
    return dispatch_hyper<bf16_t>(num_streams, streams, stream_stride, update, parts, part_stride, mix, share, read, weight,
                                  bias, eps, rms, out, rows, n_rows, width, store, stream);
  return FE_BAD_ARGUMENT;
}

// ---------------------------------------------------------------- embedding with a table of token pairs
template <typename T>
__global__ void embed_pairs_kernel(const int* __restrict__ ids, const T* __restrict__ table, const T* __restrict__ pairs,
                                   const int* __restrict__ positions, const int* __restrict__ token_seq,
                                   const int* __restrict__ cu_q, const int* __restrict__ slots,
                                   const int* __restrict__ previous, float* __restrict__ out, int H, int vocab,
                                   long long buckets, long long mul_prev, long long mul_cur, int num_slots) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 || id >= vocab) id = 0;
  long long row = buckets;                      // a sequence's first token: the table's last row
  if (positions[t] != 0) {
    const int seq = token_seq[t];
    int prev;
    if (t > cu_q[seq]) {
      prev = ids[t - 1];
    } else {
      const int slot = slots[seq];
      prev = (slot >= 0 && slot < num_slots) ? previous[slot] : 0;
    }
    if (prev < 0 || prev >= vocab) prev = 0;
    row = ((long long)prev * mul_prev + (long long)id * mul_cur) % buckets;
  }
  const T* a = table + (size_t)id * H;
  const T* b = pairs + (size_t)row * H;
  float* o = out + (size_t)t * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) o[c] = load_as_float(a + c) + load_as_float(b + c);
}

__global__ void save_last_tokens_kernel(const int* __restrict__ ids, const int* __restrict__ cu_q,
                                        const int* __restrict__ slots, int* __restrict__ previous, int num_seqs,
                                        int num_slots) {
  const int seq = blockIdx.x * blockDim.x + threadIdx.x;
  if (seq >= num_seqs) return;
  const int begin = cu_q[seq], end = cu_q[seq + 1];
  const int slot = slots[seq];
  if (end > begin && slot >= 0 && slot < num_slots) previous[slot] = ids[end - 1];
}

extern "C" int fe_embed_token_pairs(const int* ids, const void* table, const void* pairs, int dtype, const int* positions,
                                    const int* token_seq, const int* cu_q, const int* slots, int* previous, float* out,
                                    int tokens, int hidden, int vocab, long long buckets, long long mul_prev,
                                    long long mul_cur, int num_seqs, int num_slots, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (hidden <= 0 || vocab <= 0 || buckets <= 0 || mul_prev < 0 || mul_cur < 0 || num_seqs <= 0 || num_slots <= 0)
    return FE_BAD_ARGUMENT;
  const int threads = hidden >= 1024 ? 256 : 64;
  if (dtype == FE_F32)
    embed_pairs_kernel<float><<<tokens, threads, 0, stream>>>(ids, (const float*)table, (const float*)pairs, positions, token_seq,
                                                              cu_q, slots, previous, out, hidden, vocab, buckets, mul_prev,
                                                              mul_cur, num_slots);
  else if (dtype == FE_BF16)
    embed_pairs_kernel<bf16_t><<<tokens, threads, 0, stream>>>(ids, (const bf16_t*)table, (const bf16_t*)pairs, positions,
                                                               token_seq, cu_q, slots, previous, out, hidden, vocab, buckets,
                                                               mul_prev, mul_cur, num_slots);
  else
    return FE_BAD_ARGUMENT;
  // every sequence's last token, for its next step; after the kernel above has read the old ones
  save_last_tokens_kernel<<<(num_seqs + 63) / 64, 64, 0, stream>>>(ids, cu_q, slots, previous, num_seqs, num_slots);
  return fe_check_launch();
}

// ---------------------------------------------------------------- a factor on every element
__global__ void scale_kernel(float* __restrict__ x, float factor, long long count) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) x[i] *= factor;
}

extern "C" int fe_scale_rows(float* x, float factor, long long count, hipStream_t stream) {
  if (count <= 0) return FE_OK;
  scale_kernel<<<(int)((count + 255) / 256), 256, 0, stream>>>(x, factor, count);
  return fe_check_launch();
}
