// From the projection's output to queries and cached keys and values, for attention that
// normalises q and k over the whole projection: one block per token, or, in a step of few tokens, one
// per token and head.
//   q <- q / sqrt(mean over all heads and dims of q^2 + eps) * w_q      (w_q as long as q; k likewise)
//   the first R dims of every head turn by the token's position: dim i < R/2 pairs with i + R/2,
//   (a, b) -> (a c - b s, b c + a s) with c = magnitude cos(p f_i), s = magnitude sin(p f_i)
//   q into q_out [T, Hq D]; k into pages [page][kv head][slot][D]; v into pages transposed
//   [page][kv head][Dv][slot].
// With write_kv = 0 the row holds q only (a layer that reads another layer's keys and values).
// float32 inside, one rounding at the stores.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void whole_norm_rope_kernel(
    const T* __restrict__ qkv, size_t stride, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    const float* __restrict__ inv_freq, const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ block_table, int table_stride, T* __restrict__ key_pages, T* __restrict__ value_pages,
    T* __restrict__ q_out, int q_heads, int kv_heads, int D, int Dv, int R, float eps, float magnitude, int write_kv,
    int block_size, int num_blocks) {
  __shared__ float cs[128], sn[128];
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int pos = positions[t];
  const int half = R / 2;
  for (int j = tid; j < half; j += 256) {
    float s, c;
    sincosf((float)pos * inv_freq[j], &s, &c);
    cs[j] = c * magnitude;
    sn[j] = s * magnitude;
  }
  const T* row = qkv + (size_t)t * stride;
  const int q_size = q_heads * D, kv_size = kv_heads * D;
  float sq = 0.f, sk = 0.f;
  for (int e = tid; e < q_size; e += 256) {
    const float v = load_as_float(row + e);
    sq = fmaf(v, v, sq);
  }
  if (write_kv)
    for (int e = tid; e < kv_size; e += 256) {
      const float v = load_as_float(row + q_size + e);
      sk = fmaf(v, v, sk);
    }
  const float inv_q = 1.f / sqrtf(block_sum<true>(sq, scratch) / (float)q_size + eps);
  const float inv_k = write_kv ? 1.f / sqrtf(block_sum(sk, scratch) / (float)kv_size + eps) : 0.f;
  // block_sum's barriers also make cs and sn visible

  auto turned = [&](const T* x, const float* w, float inv, int e, int d) {
    float v = load_as_float(x + e) * inv * w[e];
    if (d < R) {
      const bool low = d < half;
      const int j = low ? d : d - half;
      const int pe = low ? e + half : e - half;
      const float partner = load_as_float(x + pe) * inv * w[pe];
      v = low ? v * cs[j] - partner * sn[j] : v * cs[j] + partner * sn[j];
    }
    return v;
  };

  // Units of work: the q heads, then the k heads, then the v heads.  A launch of many tokens gives a block
  // all units of its token; one of few tokens spreads them over blockIdx.y (every block forms the sums of
  // squares for itself), so that a step of a few single tokens still fills some of the chip.
  const int units = q_heads + (write_kv ? 2 * kv_heads : 0);
  int page = -1, slot = 0;
  if (write_kv) {
    const int seq = token_seq[t];
    page = block_table[(size_t)seq * table_stride + pos / block_size];
    if (page < 0 || page >= num_blocks) page = -1;
    slot = pos % block_size;
  }
  T* qrow = q_out + (size_t)t * q_size;
  const T* krow = row + q_size;
  const T* vrow = krow + kv_size;
  auto q_range = [&](int begin, int end) {
    for (int e = begin + tid; e < end; e += 256) store_from_float(qrow + e, turned(row, q_weight, inv_q, e, e % D));
  };
  auto k_range = [&](int begin, int end) {
    for (int e = begin + tid; e < end; e += 256) {
      const int h = e / D, d = e - h * D;
      store_from_float(key_pages + (((size_t)page * kv_heads + h) * block_size + slot) * D + d,
                       turned(krow, k_weight, inv_k, e, d));
    }
  };
  auto v_range = [&](int begin, int end) {
    for (int e = begin + tid; e < end; e += 256) {
      const int h = e / Dv, d = e - h * Dv;
      value_pages[(((size_t)page * kv_heads + h) * Dv + d) * block_size + slot] = vrow[e];
    }
  };
  if (gridDim.y == 1) {
    q_range(0, q_size);
    if (page >= 0) {
      k_range(0, kv_size);
      v_range(0, kv_heads * Dv);
    }
    return;
  }
  for (int unit = blockIdx.y; unit < units; unit += gridDim.y) {
    if (unit < q_heads) {
      q_range(unit * D, (unit + 1) * D);
    } else if (page >= 0 && unit < q_heads + kv_heads) {
      k_range((unit - q_heads) * D, (unit - q_heads + 1) * D);
    } else if (page >= 0) {
      v_range((unit - q_heads - kv_heads) * Dv, (unit - q_heads - kv_heads + 1) * Dv);
    }
  }
}

extern "C" int fe_whole_norm_rope_write(const void* qkv, int dtype, long long stride, const float* q_weight,
                                        const float* k_weight, const float* inv_freq, const int* positions,
                                        const int* token_seq, const int* block_table, int table_stride, void* key_pages,
                                        void* value_pages, void* q_out, int tokens, int q_heads, int kv_heads,
                                        int head_dim, int value_dim, int rotary_dim, float eps, float magnitude,
                                        int write_kv, int block_size, int num_blocks, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  const long long need = (long long)q_heads * head_dim + (write_kv ? (long long)kv_heads * (head_dim + value_dim) : 0);
  if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || value_dim <= 0 || rotary_dim < 0 || rotary_dim % 2 ||
      rotary_dim > head_dim || rotary_dim > 256 || stride < need || !(eps > 0.f) || !q_weight || (rotary_dim && !inv_freq) ||
      (write_kv && (!k_weight || !key_pages || !value_pages || !block_table || block_size <= 0 || num_blocks <= 0)))
    return FE_BAD_ARGUMENT;
  const int units = q_heads + (write_kv ? 2 * kv_heads : 0);
  const dim3 grid(tokens, tokens <= 256 ? (units < 65535 ? units : 65535) : 1);
#define LAUNCH(T)                                                                                                      \
  whole_norm_rope_kernel<T><<<grid, 256, 0, stream>>>((const T*)qkv, (size_t)stride, q_weight, k_weight, inv_freq,   \
                                                        positions, token_seq, block_table, table_stride, (T*)key_pages, \
                                                        (T*)value_pages, (T*)q_out, q_heads, kv_heads, head_dim,       \
                                                        value_dim, rotary_dim, eps, magnitude, write_kv, block_size,   \
                                                        num_blocks)
  if (dtype == FE_F32) LAUNCH(float);
  else if (dtype == FE_BF16) LAUNCH(bf16_t);
  else return FE_BAD_ARGUMENT;
#undef LAUNCH
  return fe_check_launch();
}
