// Row-wise kernels of layers that normalise their sublayers' outputs and blend a token with the
// one before it: token shift, RMSNorm of an update added into the stream, the mean of several
// normalised updates, the PolyNorm activation, and the per-head norm with weight and gate behind
// a recurrent read-out.  Statistics, norms and the stream are float32 in every mode; one rounding
// at a store into the compute dtype.  One block per row (token) unless noted; a row is read
// again from cache in the second pass, so any width works.
#include "common.h"

#define ROW_THREADS 256
#define ROW_THREADS_FEW 1024   // threads a row when a step has few rows (measured faster up to some hundred rows)
#define FEW_ROWS 512
static inline int row_threads(int rows, int width) { return rows <= FEW_ROWS && width >= 1024 ? ROW_THREADS_FEW : ROW_THREADS; }

// ---------------------------------------------------------------- token shift
// out[s][t][c] = x[t][c] + (prev[t][c] - x[t][c]) * w[s][c]; prev = x[t - 1] inside the token's
// sequence, the sequence's state row for its first token of the step.
template <typename TX, typename TO>
__global__ __launch_bounds__(ROW_THREADS_FEW) void token_shift_kernel(
    const TX* __restrict__ x, const float* __restrict__ w, const float* __restrict__ state,
    const int* __restrict__ cu_q, const int* __restrict__ token_seq, const int* __restrict__ state_slots,
    TO* __restrict__ out, int tokens, int width, int count, int slots) {
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  const bool first = cu_q[seq] == t;
  const int slot = state_slots[seq];
  const TX* row = x + (size_t)t * width;
  const TX* before = first ? row : row - width;   // never an address before the buffer
  const float* kept = state + (size_t)min(max(slot, 0), slots - 1) * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = load_as_float(row + c);
    const float p = first ? kept[c] : load_as_float(before + c);
    const float d = p - v;
    for (int s = 0; s < count; ++s)
      store_from_float(out + ((size_t)s * tokens + t) * width + c, v + d * w[(size_t)s * width + c]);
  }
}

// state[slot[s]] = x[last row of sequence s], for sequences that bring tokens.  One block per sequence.
template <typename TX>
__global__ __launch_bounds__(ROW_THREADS) void save_last_rows_kernel(
    const TX* __restrict__ x, float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, int width, int slots, int tokens) {
  const int seq = blockIdx.x;
  const int begin = cu_q[seq], end = cu_q[seq + 1];
  const int slot = state_slots[seq];
  if (end <= begin || end > tokens || slot < 0 || slot >= slots) return;
  const TX* row = x + (size_t)(end - 1) * width;
  float* kept = state + (size_t)slot * width;
  for (int c = threadIdx.x; c < width; c += ROW_THREADS) kept[c] = load_as_float(row + c);
}

extern "C" int fe_token_shift(const void* x, int x_dtype, const float* weights, const float* state, const int* cu_q,
                              const int* token_seq, const int* state_slots, void* out, int out_dtype, int tokens,
                              int width, int count, int slots, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (width <= 0 || count < 1 || count > 8 || slots < 1) return FE_BAD_ARGUMENT;
#define LAUNCH(TX, TO)                                                                                       \
  token_shift_kernel<TX, TO><<<tokens, row_threads(tokens, width), 0, stream>>>((const TX*)x, weights, state, cu_q, token_seq, \
                                                                  state_slots, (TO*)out, tokens, width, count, slots)
  if (x_dtype == FE_F32 && out_dtype == FE_F32) LAUNCH(float, float);
  else if (x_dtype == FE_F32 && out_dtype == FE_BF16) LAUNCH(float, bf16_t);
  else if (x_dtype == FE_BF16 && out_dtype == FE_BF16) LAUNCH(bf16_t, bf16_t);
  else if (x_dtype == FE_BF16 && out_dtype == FE_F32) LAUNCH(bf16_t, float);
  else return FE_BAD_ARGUMENT;
#undef LAUNCH
  return fe_check_launch();
}

extern "C" int fe_save_last_rows(const void* x, int x_dtype, float* state, const int* cu_q, const int* state_slots,
                                 int num_seqs, int width, int slots, int tokens, hipStream_t stream) {
  if (num_seqs <= 0 || tokens <= 0) return FE_OK;
  if (width <= 0 || slots < 1) return FE_BAD_ARGUMENT;
  if (x_dtype == FE_F32)
    save_last_rows_kernel<float><<<num_seqs, ROW_THREADS, 0, stream>>>((const float*)x, state, cu_q, state_slots, width, slots, tokens);
  else if (x_dtype == FE_BF16)
    save_last_rows_kernel<bf16_t><<<num_seqs, ROW_THREADS, 0, stream>>>((const bf16_t*)x, state, cu_q, state_slots, width, slots, tokens);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// ---------------------------------------------------------------- norms of updates
__device__ __forceinline__ float parts_sum(const float* p, int parts, size_t part_stride) {
  float d = p[0];
  for (int k = 1; k < parts; ++k) d += p[k * part_stride];
  return d;
}

// h[r] += u * rsqrt(mean(u^2) + eps) * w, u = the sum of the update's parts; out (if any) = new h.
// A row of up to 8 elements a thread stays in registers between the two passes (the parts are read
// once); wider rows are read again.
template <typename TO, bool HAS_OUT>
__global__ __launch_bounds__(ROW_THREADS_FEW) void rmsnorm_update_kernel(
    float* __restrict__ h, const float* __restrict__ update, int parts, size_t part_stride,
    const float* __restrict__ w, float eps, TO* __restrict__ out, int width) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * width;
  const int threads = blockDim.x;
  const bool held = width <= 8 * threads;
  float u[8];
  float ss = 0.f;
  if (held) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = threadIdx.x + j * threads;
      u[j] = c < width ? parts_sum(update + base + c, parts, part_stride) : 0.f;
      ss += u[j] * u[j];
    }
  } else {
    for (int c = threadIdx.x; c < width; c += threads) {
      const float v = parts_sum(update + base + c, parts, part_stride);
      ss += v * v;
    }
  }
  ss = block_sum<true>(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
  if (held) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = threadIdx.x + j * threads;
      if (c < width) {
        const float v = h[base + c] + u[j] * inv * w[c];
        h[base + c] = v;
        if (HAS_OUT) store_from_float(out + base + c, v);
      }
    }
  } else {
    for (int c = threadIdx.x; c < width; c += threads) {
      const float v = h[base + c] + parts_sum(update + base + c, parts, part_stride) * inv * w[c];
      h[base + c] = v;
      if (HAS_OUT) store_from_float(out + base + c, v);
    }
  }
}

extern "C" int fe_rmsnorm_update(float* h, const float* update, int parts, long long part_stride, const float* w,
                                 float eps, void* out, int out_dtype, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (width <= 0 || parts < 1 || parts > 64 || !(eps > 0.f)) return FE_BAD_ARGUMENT;
  if (out == nullptr || out_dtype < 0)
    rmsnorm_update_kernel<float, false><<<rows, row_threads(rows, width), 0, stream>>>(h, update, parts, (size_t)part_stride, w, eps, nullptr, width);
  else if (out_dtype == FE_F32)
    rmsnorm_update_kernel<float, true><<<rows, row_threads(rows, width), 0, stream>>>(h, update, parts, (size_t)part_stride, w, eps, (float*)out, width);
  else if (out_dtype == FE_BF16)
    rmsnorm_update_kernel<bf16_t, true><<<rows, row_threads(rows, width), 0, stream>>>(h, update, parts, (size_t)part_stride, w, eps, (bf16_t*)out, width);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// h[r] += factor * (u - mean(u)) * rsqrt(var(u) + eps) * w, u = the sum of the update's parts, var the mean
// of the squared deviations; out (if any) = new h.  A row of up to 8 elements a thread stays in
// registers between the three passes; wider rows are read again.
template <typename TO, bool HAS_OUT>
__global__ __launch_bounds__(ROW_THREADS_FEW) void layernorm_update_kernel(
    float* __restrict__ h, const float* __restrict__ update, int parts, size_t part_stride,
    const float* __restrict__ w, float eps, float factor, TO* __restrict__ out, int width) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * width;
  const int threads = blockDim.x;
  const bool held = width <= 8 * threads;
  float u[8];
  float sum = 0.f;
  if (held) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = threadIdx.x + j * threads;
      u[j] = c < width ? parts_sum(update + base + c, parts, part_stride) : 0.f;
      sum += u[j];
    }
  } else {
    for (int c = threadIdx.x; c < width; c += threads) sum += parts_sum(update + base + c, parts, part_stride);
  }
  const float mean = block_sum<true>(sum, scratch) / (float)width;
  float ss = 0.f;
  if (held) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = threadIdx.x + j * threads;
      const float d = c < width ? u[j] - mean : 0.f;
      ss += d * d;
    }
  } else {
    for (int c = threadIdx.x; c < width; c += threads) {
      const float d = parts_sum(update + base + c, parts, part_stride) - mean;
      ss += d * d;
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps) * factor;
  if (held) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int c = threadIdx.x + j * threads;
      if (c < width) {
        const float v = h[base + c] + (u[j] - mean) * inv * w[c];
        h[base + c] = v;
        if (HAS_OUT) store_from_float(out + base + c, v);
      }
    }
  } else {
    for (int c = threadIdx.x; c < width; c += threads) {
      const float v = h[base + c] + (parts_sum(update + base + c, parts, part_stride) - mean) * inv * w[c];
      h[base + c] = v;
      if (HAS_OUT) store_from_float(out + base + c, v);
    }
  }
}

extern "C" int fe_layernorm_update(float* h, const float* update, int parts, long long part_stride, const float* w,
                                   float eps, float factor, void* out, int out_dtype, int rows, int width,
                                   hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (width <= 0 || parts < 1 || parts > 64 || !(eps > 0.f)) return FE_BAD_ARGUMENT;
  const int threads = row_threads(rows, width);
  if (out == nullptr || out_dtype < 0)
    layernorm_update_kernel<float, false><<<rows, threads, 0, stream>>>(h, update, parts, (size_t)part_stride, w, eps, factor, nullptr, width);
  else if (out_dtype == FE_F32)
    layernorm_update_kernel<float, true><<<rows, threads, 0, stream>>>(h, update, parts, (size_t)part_stride, w, eps, factor, (float*)out, width);
  else if (out_dtype == FE_BF16)
    layernorm_update_kernel<bf16_t, true><<<rows, threads, 0, stream>>>(h, update, parts, (size_t)part_stride, w, eps, factor, (bf16_t*)out, width);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// A norm behind a sublayer and the norm before the next one in one pass over the row:
//   v = h[s] + u * rsqrt(mean(u^2) + eps) * w        (u = the sum of the update's parts; written back to h if `store`)
//   out[r] = v * rsqrt(mean(v^2) + eps_next) * w_next,  s = rows[r] or r.
// The row (up to 8 elements a thread) stays in registers between the three passes.  VEC 4: a thread's
// elements are two runs of four neighbours (16-byte loads and stores; the width a multiple of four).
template <typename TO, int VEC>
__global__ __launch_bounds__(ROW_THREADS_FEW) void rmsnorm_update_norm_kernel(
    float* __restrict__ h, const float* __restrict__ update, int parts, size_t part_stride,
    const float* __restrict__ w, float eps, const float* __restrict__ w_next, float eps_next, TO* __restrict__ out,
    const int* __restrict__ rows, int store, int width) {
  __shared__ float scratch[16];
  const size_t base = (size_t)(rows ? rows[blockIdx.x] : (int)blockIdx.x) * width;
  const size_t out_base = (size_t)blockIdx.x * width;
  const int threads = blockDim.x;
  constexpr int RUNS = 8 / VEC;
  float u[8];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < RUNS; ++j) {
    const int c = (threadIdx.x + j * threads) * VEC;
    if constexpr (VEC == 4) {
      float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
      if (c < width) {
        sum = *reinterpret_cast<const float4*>(update + base + c);
        for (int k = 1; k < parts; ++k) {
          const float4 more = *reinterpret_cast<const float4*>(update + k * part_stride + base + c);
          sum.x += more.x; sum.y += more.y; sum.z += more.z; sum.w += more.w;
        }
      }
      u[4 * j] = sum.x; u[4 * j + 1] = sum.y; u[4 * j + 2] = sum.z; u[4 * j + 3] = sum.w;
      ss += sum.x * sum.x + sum.y * sum.y + sum.z * sum.z + sum.w * sum.w;
    } else {
      u[j] = c < width ? parts_sum(update + base + c, parts, part_stride) : 0.f;
      ss += u[j] * u[j];
    }
  }
  ss = block_sum<true>(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
  float ss_next = 0.f;
#pragma unroll
  for (int j = 0; j < RUNS; ++j) {
    const int c = (threadIdx.x + j * threads) * VEC;
    if (c < width) {
      if constexpr (VEC == 4) {
        const float4 before = *reinterpret_cast<const float4*>(h + base + c);
        const float4 weight = *reinterpret_cast<const float4*>(w + c);
        float4 v;
        v.x = before.x + u[4 * j] * inv * weight.x;
        v.y = before.y + u[4 * j + 1] * inv * weight.y;
        v.z = before.z + u[4 * j + 2] * inv * weight.z;
        v.w = before.w + u[4 * j + 3] * inv * weight.w;
        if (store) *reinterpret_cast<float4*>(h + base + c) = v;
        u[4 * j] = v.x; u[4 * j + 1] = v.y; u[4 * j + 2] = v.z; u[4 * j + 3] = v.w;
        ss_next += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      } else {
        u[j] = h[base + c] + u[j] * inv * w[c];
        if (store) h[base + c] = u[j];
        ss_next += u[j] * u[j];
      }
    }
  }
  ss_next = block_sum(ss_next, scratch);
  const float inv_next = rsqrtf(ss_next / (float)width + eps_next);
#pragma unroll
  for (int j = 0; j < RUNS; ++j) {
    const int c = (threadIdx.x + j * threads) * VEC;
    if (c < width) {
      if constexpr (VEC == 4) {
        const float4 weight = *reinterpret_cast<const float4*>(w_next + c);
        struct alignas(sizeof(TO) * 4) Pack { TO e[4]; } pack;
        store_from_float(&pack.e[0], u[4 * j] * inv_next * weight.x);
        store_from_float(&pack.e[1], u[4 * j + 1] * inv_next * weight.y);
        store_from_float(&pack.e[2], u[4 * j + 2] * inv_next * weight.z);
        store_from_float(&pack.e[3], u[4 * j + 3] * inv_next * weight.w);
        *reinterpret_cast<Pack*>(out + out_base + c) = pack;
      } else {
        store_from_float(out + out_base + c, u[j] * inv_next * w_next[c]);
      }
    }
  }
}

// rows: indices of the rows to take (int32 [count]) or null for all `count` rows in order; with a row list
// nothing is written back (store must be 0: rows may repeat).  Rows up to 8,192 wide (8 elements a thread).
extern "C" int fe_rmsnorm_update_norm(float* h, const float* update, int parts, long long part_stride, const float* w,
                                      float eps, const float* w_next, float eps_next, void* out, int out_dtype,
                                      const int* rows, int store, int count, int width, hipStream_t stream) {
  if (count <= 0) return FE_OK;
  const int threads = width > 8 * ROW_THREADS ? ROW_THREADS_FEW : row_threads(count, width);
  if (width <= 0 || width > 8 * threads || parts < 1 || parts > 64 || !(eps > 0.f) || !(eps_next > 0.f) || !out ||
      (rows && store) || (out_dtype != FE_F32 && out_dtype != FE_BF16))
    return FE_BAD_ARGUMENT;
  const bool wide = width % 4 == 0 && part_stride % 4 == 0 && (uintptr_t)h % 16 == 0 && (uintptr_t)update % 16 == 0 &&
                    (uintptr_t)w % 16 == 0 && (uintptr_t)w_next % 16 == 0 && (uintptr_t)out % 16 == 0;
#define LAUNCH(TO, VEC)                                                                                               \
  rmsnorm_update_norm_kernel<TO, VEC><<<count, threads, 0, stream>>>(h, update, parts, (size_t)part_stride, w, eps, w_next, \
                                                                     eps_next, (TO*)out, rows, store, width)
  if (out_dtype == FE_F32) {
    if (wide) LAUNCH(float, 4); else LAUNCH(float, 1);
  } else {
    if (wide) LAUNCH(bf16_t, 4); else LAUNCH(bf16_t, 1);
  }
#undef LAUNCH
  return fe_check_launch();
}

// out[r] = (1 / n) sum_b u_b * rsqrt(mean(u_b^2) + eps) * w[b]
struct MeanInputs {
  const float* u[4];
  int parts[4];
};

__global__ __launch_bounds__(ROW_THREADS_FEW) void rmsnorm_mean_kernel(MeanInputs in, int count, size_t part_stride,
                                                                   const float* __restrict__ w, float eps,
                                                                   float* __restrict__ out, int width) {
  __shared__ float scratch[4][16];
  const size_t base = (size_t)blockIdx.x * width;
  float inv[4];
  for (int b = 0; b < count; ++b) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      const float u = parts_sum(in.u[b] + base + c, in.parts[b], part_stride);
      ss += u * u;
    }
    ss = block_sum<true>(ss, scratch[b]);
    inv[b] = rsqrtf(ss / (float)width + eps);
  }
  const float share = 1.f / (float)count;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float total = 0.f;
    for (int b = 0; b < count; ++b)
      total += parts_sum(in.u[b] + base + c, in.parts[b], part_stride) * inv[b] * w[(size_t)b * width + c];
    out[base + c] = total * share;
  }
}

extern "C" int fe_rmsnorm_mean(const float* u0, const float* u1, const float* u2, const float* u3, int p0, int p1,
                               int p2, int p3, int count, long long part_stride, const float* w, float eps,
                               float* out, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (width <= 0 || count < 1 || count > 4 || !(eps > 0.f)) return FE_BAD_ARGUMENT;
  MeanInputs in = {{u0, u1, u2, u3}, {p0, p1, p2, p3}};
  for (int b = 0; b < count; ++b)
    if (in.u[b] == nullptr || in.parts[b] < 1 || in.parts[b] > 64) return FE_BAD_ARGUMENT;
  rmsnorm_mean_kernel<<<rows, row_threads(rows, width), 0, stream>>>(in, count, (size_t)part_stride, w, eps, out, width);
  return fe_check_launch();
}

// ---------------------------------------------------------------- PolyNorm
// out = a z/rms(z) + b z^2/rms(z^2) + c z^3/rms(z^3) + e over a row
template <typename T>
__global__ __launch_bounds__(ROW_THREADS_FEW) void polynorm_kernel(const T* __restrict__ z, const float* __restrict__ coeff,
                                                               float eps, T* __restrict__ out, int width) {
  __shared__ float scratch[3][16];
  const size_t base = (size_t)blockIdx.x * width;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = load_as_float(z + base + c);
    const float v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  s1 = block_sum<true>(s1, scratch[0]);
  s2 = block_sum<true>(s2, scratch[1]);
  s3 = block_sum<true>(s3, scratch[2]);
  const float n = (float)width;
  const float a = coeff[0] * rsqrtf(s1 / n + eps), b = coeff[1] * rsqrtf(s2 / n + eps),
              c3 = coeff[2] * rsqrtf(s3 / n + eps), e = coeff[3];
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = load_as_float(z + base + c);
    const float v2 = v * v;
    store_from_float(out + base + c, a * v + b * v2 + c3 * (v2 * v) + e);
  }
}

extern "C" int fe_polynorm(const void* z, int dtype, const float* coeff, float eps, void* out, int rows, int width,
                           hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (width <= 0 || !(eps > 0.f)) return FE_BAD_ARGUMENT;
  if (dtype == FE_F32)
    polynorm_kernel<float><<<rows, row_threads(rows, width), 0, stream>>>((const float*)z, coeff, eps, (float*)out, width);
  else if (dtype == FE_BF16)
    polynorm_kernel<bf16_t><<<rows, row_threads(rows, width), 0, stream>>>((const bf16_t*)z, coeff, eps, (bf16_t*)out, width);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// ---------------------------------------------------------------- bias of an update
// update[r][c] += bias[c] for the first `rows * width` elements (the first part of an update in parts).
__global__ void add_bias_kernel(float* __restrict__ update, const float* __restrict__ bias, long long count, int width) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) update[i] += bias[i % width];
}

extern "C" int fe_add_bias(float* update, const float* bias, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (width <= 0) return FE_BAD_ARGUMENT;
  const long long count = (long long)rows * width;
  add_bias_kernel<<<(int)((count + 255) / 256), 256, 0, stream>>>(update, bias, count, width);
  return fe_check_launch();
}

// ---------------------------------------------------------------- output gate
// out[t][c] *= sigmoid(gate[t][c / share]), gate rows `gate_stride` elements apart; `share` consecutive
// outputs take one gate (1: a gate per element; a head's width: a gate per head)
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ out, const T* __restrict__ gate, size_t gate_stride, int width,
                                    long long count, int share) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const long long t = i / width;
  const int c = (int)(i - t * width);
  const float g = load_as_float(gate + (size_t)t * gate_stride + c / share);
  store_from_float(out + i, load_as_float(out + i) / (1.f + expf(-g)));
}

extern "C" int fe_sigmoid_gate(void* out, const void* gate, long long gate_stride, int dtype, int rows, int width,
                               int share, hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (width <= 0 || share < 1 || width % share || gate_stride < width / share) return FE_BAD_ARGUMENT;
  const long long count = (long long)rows * width;
  const int blocks = (int)((count + 255) / 256);
  if (dtype == FE_F32) sigmoid_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gate, (size_t)gate_stride, width, count, share);
  else if (dtype == FE_BF16) sigmoid_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gate, (size_t)gate_stride, width, count, share);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// ---------------------------------------------------------------- tanh in place
template <typename T>
__global__ void tanh_kernel(T* __restrict__ x, long long count) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) store_from_float(x + i, tanhf(load_as_float(x + i)));
}

extern "C" int fe_tanh_rows(void* x, int dtype, long long count, hipStream_t stream) {
  if (count <= 0) return FE_OK;
  const int blocks = (int)((count + 255) / 256);
  if (dtype == FE_F32) tanh_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, count);
  else if (dtype == FE_BF16) tanh_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, count);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// The square of relu over every element, float32 inside.
template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ x, T* __restrict__ out, long long count) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const float v = fmaxf(load_as_float(x + i), 0.f);
  store_from_float(out + i, v * v);
}

extern "C" int fe_relu_squared(const void* x, void* out, int dtype, long long count, hipStream_t stream) {
  if (count <= 0) return FE_OK;
  const long long blocks = (count + 255) / 256;
  if (blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  if (dtype == FE_F32) relu_squared_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((const float*)x, (float*)out, count);
  else if (dtype == FE_BF16) relu_squared_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, count);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// An activation over every element, float32 inside: 0 the square of relu, 1 the gelu with the error
// function, 0.5 z (1 + erf(z / sqrt 2)), 2 its tanh form, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))).
template <typename T, int KIND>
__global__ void activate_kernel(const T* __restrict__ x, T* __restrict__ out, long long count) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const float z = load_as_float(x + i);
  float v;
  if (KIND == 0) {
    v = fmaxf(z, 0.f);
    v = v * v;
  } else if (KIND == 1) {
    v = 0.5f * z * (1.f + erff(z * 0.70710678118654752440f));
  } else {
    v = 0.5f * z * (1.f + tanhf(0.79788456080286535588f * (z + 0.044715f * z * z * z)));
  }
  store_from_float(out + i, v);
}

extern "C" int fe_activate(const void* x, void* out, int dtype, long long count, int kind, hipStream_t stream) {
  if (count <= 0) return FE_OK;
  const long long blocks = (count + 255) / 256;
  if (blocks > 0x7fffffffLL || kind < 0 || kind > 2 || (dtype != FE_F32 && dtype != FE_BF16)) return FE_BAD_ARGUMENT;
#define LAUNCH(T, KIND) activate_kernel<T, KIND><<<(unsigned)blocks, 256, 0, stream>>>((const T*)x, (T*)out, count)
  if (dtype == FE_F32) {
    if (kind == 0) LAUNCH(float, 0); else if (kind == 1) LAUNCH(float, 1); else LAUNCH(float, 2);
  } else {
    if (kind == 0) LAUNCH(bf16_t, 0); else if (kind == 1) LAUNCH(bf16_t, 1); else LAUNCH(bf16_t, 2);
  }
#undef LAUNCH
  return fe_check_launch();
}

// update[p][t][c] *= sigmoid(gate[t * gate_stride]): one gate a row, float32, over every part of an update.
__global__ void gate_rows_kernel(float* __restrict__ update, const float* __restrict__ gate, size_t gate_stride,
                                 int rows, int width, long long count) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const long long t = (i / width) % rows;
  update[i] *= 1.f / (1.f + expf(-gate[(size_t)t * gate_stride]));
}

extern "C" int fe_gate_rows(float* update, int parts, const float* gate, long long gate_stride, int rows, int width,
                            hipStream_t stream) {
  if (rows <= 0) return FE_OK;
  if (width <= 0 || parts < 1 || gate_stride < 1) return FE_BAD_ARGUMENT;
  const long long count = (long long)parts * rows * width;
  const long long blocks = (count + 255) / 256;
  if (blocks > 0x7fffffffLL) return FE_BAD_ARGUMENT;
  gate_rows_kernel<<<(unsigned)blocks, 256, 0, stream>>>(update, gate, (size_t)gate_stride, rows, width, count);
  return fe_check_launch();
}

// ---------------------------------------------------------------- per-head norm, weight and gate
// One wave per (token, head): y = o[:dim] (divided by max(|o[dim]|, floor) + 1e-6 with a normaliser
// column), y / rms(y) * weight * act(gate).
__device__ __forceinline__ float gate_act(float g, int act) {
  if (act == 1) return g / (1.f + expf(-g));
  if (act == 2) return 1.f / (1.f + expf(-g));
  return 1.f;
}

template <typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(
    const float* __restrict__ o, const float* __restrict__ weight, int weight_len, const TO* __restrict__ gate,
    size_t gate_stride, TO* __restrict__ out, const float* __restrict__ floor_, int tokens, int heads, int dim,
    int extra, float eps, int act) {
  const int lane = threadIdx.x & 63;
  const long long pair = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= (long long)tokens * heads) return;
  const int t = (int)(pair / heads), h = (int)(pair - (long long)t * heads);
  const float* row = o + (size_t)pair * (dim + extra);
  float scale = 1.f;
  if (extra) scale = 1.f / (fmaxf(fabsf(row[dim]), floor_[pair]) + 1e-6f);
  float ss = 0.f;
  for (int c = lane; c < dim; c += 64) {
    const float v = row[c] * scale;
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)dim + eps) * scale;
  for (int c = lane; c < dim; c += 64) {
    float v = row[c] * inv;
    if (weight) v *= weight[weight_len == dim ? c : h * dim + c];
    if (gate) v *= gate_act(load_as_float(gate + (size_t)t * gate_stride + h * dim + c), act);
    store_from_float(out + ((size_t)t * heads + h) * dim + c, v);
  }
}

extern "C" int fe_head_norm_gate(const float* o, const float* weight, int weight_len, const void* gate,
                                 long long gate_stride, void* out, int out_dtype, const float* floor_, int tokens,
                                 int heads, int dim, int extra, float eps, int act, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (heads <= 0 || dim <= 0 || extra < 0 || extra > 1 || !(eps > 0.f) || act < 0 || act > 2) return FE_BAD_ARGUMENT;
  if (weight && weight_len != dim && weight_len != heads * dim) return FE_BAD_ARGUMENT;
  if (extra && floor_ == nullptr) return FE_BAD_ARGUMENT;
  const long long pairs = (long long)tokens * heads;
  const int blocks = (int)((pairs + 3) / 4);
  if (out_dtype == FE_F32)
    head_norm_gate_kernel<float><<<blocks, 256, 0, stream>>>(o, weight, weight_len, (const float*)gate, (size_t)gate_stride,
                                                              (float*)out, floor_, tokens, heads, dim, extra, eps, act);
  else if (out_dtype == FE_BF16)
    head_norm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(o, weight, weight_len, (const bf16_t*)gate, (size_t)gate_stride,
                                                               (bf16_t*)out, floor_, tokens, heads, dim, extra, eps, act);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}
