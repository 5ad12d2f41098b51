// From the fused q/k/v projection to queries and cached keys and values, for attention whose
// projections pass a short causal convolution over time:
//   y_t[c] = sum_j w[c][j] * u_(t - taps + 1 + j)[c]        (rows before the sequence's start: zeros)
// then q and k heads are rotated (first rotary_dim dims, dim i pairs with i + rotary_dim / 2,
// angle = position * inv_freq[i]) and, if asked, divided by their root mean square (no weight);
// q goes to its own buffer, k and v into their pages (values transposed: [dim][slot]).
// Rows of a sequence that earlier steps brought come from the sequence's state slot, which holds
// its last taps - 1 projected rows; a second kernel moves the state on after the first has read it.
// The projection's bias (float32, one entry per q, k and v channel, or none) is added here, to the
// rows as they are loaded, so that the product before this kernel has none; the state holds rows
// with their bias.  One wave per token and head; everything between the loads and the stores is float32.
// The unit norm may carry a weight per dim, one for q heads and one for k heads, shared by the heads
// (an RMS norm); with `norm_first` the norm comes before the rotation instead of behind it.
// Values may lean on another layer's values of the same tokens: v <- (1 - mix) v + mix * v_from
// (v_from [T, kv_heads * value_dim], dense), after the bias and the convolution and before the page
// write; a layer that others lean on leaves its values, as stored, in v_keep (same shape).
#include "common.h"

#define CR_THREADS 256
#define CR_HEAD_MAX 256

// One wave per (token, head): q heads, then k heads, then v heads.
template <typename T>
__global__ __launch_bounds__(64) void conv_rope_norm_write_kernel(
    const T* __restrict__ qkv, size_t qkv_stride, const float* __restrict__ bias, const float* __restrict__ conv_w,
    const float* __restrict__ conv_state, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ token_seq, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ key_pages, T* __restrict__ value_pages, T* __restrict__ q_out, int q_heads, int kv_heads,
    int head_dim, int value_dim, int rotary_dim, float eps, int unit_norm, int taps, int block_size,
    int num_blocks, int slots, const T* __restrict__ v_from, float v_mix, T* __restrict__ v_keep,
    const float* __restrict__ norm_wq, const float* __restrict__ norm_wk, int norm_first) {
  __shared__ float y[CR_HEAD_MAX];
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int seq = token_seq[t];
  const int begin = cu_q[seq];
  const int pos = positions[t];
  const int q_size = q_heads * head_dim, k_size = kv_heads * head_dim, v_size = kv_heads * value_dim;
  const int channels = q_size + k_size + v_size;
  const bool is_q = head < q_heads, is_v = head >= q_heads + kv_heads;
  const int n = is_v ? value_dim : head_dim;
  const int first = is_q ? head * head_dim
                         : (is_v ? q_size + k_size + (head - q_heads - kv_heads) * value_dim : q_size + (head - q_heads) * head_dim);

  // 1. the head's channels: bias, convolution over the rows of this step and of the state
  const int slot = taps > 1 ? min(max(state_slots[seq], 0), slots - 1) : 0;
  const float* kept = taps > 1 ? conv_state + (size_t)slot * (taps - 1) * channels : nullptr;    // one tap reads no earlier row
  for (int d = lane; d < n; d += 64) {
    const int c = first + d;
    const float b = bias ? bias[c] : 0.f;
    float acc;
    if (taps > 0) {
      acc = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int row = t - (taps - 1) + j;          // a row of this step, or of the state if before `begin`
        const float u = row >= begin ? load_as_float(qkv + (size_t)row * qkv_stride + c) + b
                                     : kept[(size_t)(taps - 1 - (begin - row)) * channels + c];
        acc = fmaf(conv_w[(size_t)c * taps + j], u, acc);
      }
    } else {
      acc = load_as_float(qkv + (size_t)t * qkv_stride + c) + b;
    }
    y[d] = acc;
  }
  __syncthreads();

  const int page = block_table[(size_t)seq * table_stride + pos / block_size];
  const int place = pos % block_size;
  const bool paged = page >= 0 && page < num_blocks;
  if (is_v) {
    const int hv = head - q_heads - kv_heads;
    const size_t dense = (size_t)t * v_size + (size_t)hv * value_dim;
    for (int d = lane; d < n; d += 64) {
      float v = y[d];
      if (v_from) v = (1.f - v_mix) * v + v_mix * load_as_float(v_from + dense + d);
      if (v_keep) store_from_float(v_keep + dense + d, v);
      if (paged) store_from_float(value_pages + (((size_t)page * kv_heads + hv) * value_dim + d) * block_size + place, v);
    }
    return;
  }

  // 2. the norm where it comes first; rotation, a pair per lane
  const float* norm_w = is_q ? norm_wq : norm_wk;
  auto unit = [&]() {
    float ss = 0.f;
    for (int d = lane; d < n; d += 64) ss += y[d] * y[d];
    ss = wave_sum(ss);
    return rsqrtf(ss / (float)head_dim + eps);
  };
  if (unit_norm && norm_first) {
    const float inv = unit();
    for (int d = lane; d < n; d += 64) y[d] = y[d] * inv * (norm_w ? norm_w[d] : 1.f);
    __syncthreads();
  }
  const int half = rotary_dim / 2;
  for (int i = lane; i < half; i += 64) {
    float sn, cs;
    sincosf((float)pos * inv_freq[i], &sn, &cs);
    const float a = y[i], b = y[i + half];
    y[i] = a * cs - b * sn;
    y[i + half] = b * cs + a * sn;
  }
  __syncthreads();

  // 3. the norm behind the rotation, and the store
  float inv = 1.f;
  const bool late = unit_norm && !norm_first;
  if (late) inv = unit();
  if (is_q) {
    T* dst = q_out + (size_t)t * q_size + head * head_dim;
    for (int d = lane; d < n; d += 64) store_from_float(dst + d, y[d] * inv * (late && norm_w ? norm_w[d] : 1.f));
  } else if (paged) {
    T* dst = key_pages + (((size_t)page * kv_heads + (head - q_heads)) * block_size + place) * head_dim;
    for (int d = lane; d < n; d += 64) store_from_float(dst + d, y[d] * inv * (late && norm_w ? norm_w[d] : 1.f));
  }
}

// The state after the step: the last taps - 1 projected rows of every sequence that brought tokens.
template <typename T>
__global__ __launch_bounds__(CR_THREADS) void conv_state_update_kernel(
    const T* __restrict__ qkv, size_t qkv_stride, const float* __restrict__ bias, float* __restrict__ conv_state,
    const int* __restrict__ cu_q, const int* __restrict__ state_slots, int channels, int taps, int slots, int tokens) {
  const int seq = blockIdx.y;
  const int begin = cu_q[seq], end = cu_q[seq + 1];
  const int slot = state_slots[seq];
  const int c = blockIdx.x * CR_THREADS + threadIdx.x;
  if (end <= begin || end > tokens || slot < 0 || slot >= slots || c >= channels) return;
  const int n = end - begin;
  float* kept = conv_state + (size_t)slot * (taps - 1) * channels;
  float next[7];
#pragma unroll
  for (int j = 0; j < 7; ++j) {
    if (j < taps - 1) {
      const int r = n - (taps - 1) + j;      // relative to the step's first row
      next[j] = r >= 0 ? load_as_float(qkv + (size_t)(begin + r) * qkv_stride + c) + (bias ? bias[c] : 0.f)
                       : kept[(size_t)(taps - 1 + r) * channels + c];
    }
  }
#pragma unroll
  for (int j = 0; j < 7; ++j)
    if (j < taps - 1) kept[(size_t)j * channels + c] = next[j];
}

extern "C" int fe_conv_rope_norm_write(const void* qkv, int dtype, long long qkv_stride, const float* bias, const float* conv_w,
                                       const float* conv_state, const float* inv_freq, const int* positions,
                                       const int* token_seq, const int* cu_q, const int* state_slots,
                                       const int* block_table, int table_stride, void* key_pages, void* value_pages,
                                       void* q_out, int tokens, int q_heads, int kv_heads, int head_dim, int value_dim,
                                       int rotary_dim, float eps, int unit_norm, int taps, int block_size,
                                       int num_blocks, int slots, const void* v_from, float v_mix, void* v_keep,
                                       const float* norm_wq, const float* norm_wk, int norm_first, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || value_dim <= 0 || block_size <= 0 || num_blocks <= 0)
    return FE_BAD_ARGUMENT;
  if (rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2 || (rotary_dim && !inv_freq)) return FE_BAD_ARGUMENT;
  if (taps < 0 || taps > 8 || (taps && !conv_w) || (taps > 1 && (!conv_state || slots < 1))) return FE_BAD_ARGUMENT;
  if (unit_norm && !(eps > 0.f)) return FE_BAD_ARGUMENT;
  if (!unit_norm && (norm_wq || norm_wk || norm_first)) return FE_BAD_ARGUMENT;
  const long long channels = (long long)(q_heads + kv_heads) * head_dim + (long long)kv_heads * value_dim;
  if (head_dim > CR_HEAD_MAX || value_dim > CR_HEAD_MAX || qkv_stride < channels || q_heads + 2 * kv_heads > 65535)
    return FE_BAD_ARGUMENT;      // a head lives in LDS
  const dim3 grid(tokens, q_heads + 2 * kv_heads);
#define LAUNCH(T)                                                                                              \
  conv_rope_norm_write_kernel<T><<<grid, 64, 0, stream>>>(                                         \
      (const T*)qkv, (size_t)qkv_stride, bias, conv_w, conv_state, inv_freq, positions, token_seq, cu_q, state_slots, \
      block_table, table_stride, (T*)key_pages, (T*)value_pages, (T*)q_out, q_heads, kv_heads, head_dim,       \
      value_dim, rotary_dim, eps, unit_norm, taps, block_size, num_blocks, slots, (const T*)v_from, v_mix, (T*)v_keep, \
      norm_wq, norm_wk, norm_first)
  if (dtype == FE_F32) LAUNCH(float);
  else if (dtype == FE_BF16) LAUNCH(bf16_t);
  else return FE_BAD_ARGUMENT;
#undef LAUNCH
  return fe_check_launch();
}

extern "C" int fe_conv_state_update(const void* qkv, int dtype, long long qkv_stride, const float* bias, float* conv_state,
                                    const int* cu_q, const int* state_slots, int num_seqs, int channels, int taps,
                                    int slots, int tokens, hipStream_t stream) {
  if (num_seqs <= 0 || tokens <= 0) return FE_OK;
  if (channels <= 0 || taps < 2 || taps > 8 || slots < 1 || qkv_stride < channels) return FE_BAD_ARGUMENT;
  const dim3 grid((channels + CR_THREADS - 1) / CR_THREADS, num_seqs);
  if (dtype == FE_F32)
    conv_state_update_kernel<float><<<grid, CR_THREADS, 0, stream>>>((const float*)qkv, (size_t)qkv_stride, bias, conv_state,
                                                                     cu_q, state_slots, channels, taps, slots, tokens);
  else if (dtype == FE_BF16)
    conv_state_update_kernel<bf16_t><<<grid, CR_THREADS, 0, stream>>>((const bf16_t*)qkv, (size_t)qkv_stride, bias, conv_state,
                                                                      cu_q, state_slots, channels, taps, slots, tokens);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}
