// Attention through a latent: what lies between its products.
//
//   fe_latent_norm_rope_write: from the fused down-projections of a token, x = [a | b | r] (float32: a of
//       q_rank, b of kv_rank, r of rot_dim entries), the query latent a / rms(a) * wq into cq [T, q_rank] and,
//       for a layer that caches, the token's cache row [b / rms(b) * wkv | rotate(r)] into its page
//       (key pages [page][1][slot][kv_rank + rot_dim]) and, where the cache keeps values, the normed b a
//       second time into the transposed value pages ([page][1][kv_rank][slot], the layout the matrix-core
//       attention reads its second operand in).  The rotation turns the first rotary_dim dims
//       of r, dim i with dim i + rotary_dim / 2, by the angle position * inv_freq[i]; the rest pass.
//   fe_latent_query_pack: the attention's query rows [T, heads, kv_rank + rot_dim] from the queries taken
//       through the key up-projection (qa [heads, T, kv_rank], the result of a batched product) and
//       the rotated part of every head of q [T, heads, dim + rot_dim], rotated here.
// Norms, angles and rotations are float32, one rounding at the stores.
#include "common.h"

#define LT_THREADS 256

template <typename T>
__global__ __launch_bounds__(LT_THREADS) void latent_norm_rope_write_kernel(
    const float* __restrict__ x, size_t stride, int q_rank, int kv_rank, int rot_dim, int rotary_dim,
    const float* __restrict__ wq, const float* __restrict__ wkv, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ token_seq, const int* __restrict__ block_table,
    int table_stride, T* __restrict__ key_pages, T* __restrict__ value_pages, T* __restrict__ cq, float eps,
    int block_size, int num_blocks, int write_kv) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* row = x + (size_t)t * stride;
  float ss = 0.f;
  for (int c = tid; c < q_rank; c += LT_THREADS) ss += row[c] * row[c];
  ss = block_sum<true>(ss, scratch);
  const float inv_q = rsqrtf(ss / (float)q_rank + eps);
  for (int c = tid; c < q_rank; c += LT_THREADS) store_from_float(cq + (size_t)t * q_rank + c, row[c] * inv_q * wq[c]);
  if (!write_kv) return;

  const float* b = row + q_rank;
  float sb = 0.f;
  for (int c = tid; c < kv_rank; c += LT_THREADS) sb += b[c] * b[c];
  sb = block_sum(sb, scratch);
  const float inv_b = rsqrtf(sb / (float)kv_rank + eps);
  const int pos = positions[t];
  const int page = block_table[(size_t)token_seq[t] * table_stride + pos / block_size];
  if (page < 0 || page >= num_blocks) return;
  T* dst = key_pages + ((size_t)page * block_size + pos % block_size) * (kv_rank + rot_dim);
  T* vdst = value_pages ? value_pages + (size_t)page * kv_rank * block_size + pos % block_size : nullptr;
  for (int c = tid; c < kv_rank; c += LT_THREADS) {
    const float v = b[c] * inv_b * wkv[c];
    store_from_float(dst + c, v);
    if (vdst) store_from_float(vdst + (size_t)c * block_size, v);
  }
  const float* r = b + kv_rank;
  const int half = rotary_dim / 2;
  for (int i = tid; i < half; i += LT_THREADS) {
    float sn, cs;
    sincosf((float)pos * inv_freq[i], &sn, &cs);
    const float u = r[i], v = r[i + half];
    store_from_float(dst + kv_rank + i, u * cs - v * sn);
    store_from_float(dst + kv_rank + i + half, v * cs + u * sn);
  }
  for (int c = rotary_dim + tid; c < rot_dim; c += LT_THREADS) store_from_float(dst + kv_rank + c, r[c]);
}

extern "C" int fe_latent_norm_rope_write(const float* x, long long stride, int q_rank, int kv_rank, int rot_dim,
                                         int rotary_dim, const float* wq, const float* wkv, const float* inv_freq,
                                         const int* positions, const int* token_seq, const int* block_table,
                                         int table_stride, void* key_pages, void* value_pages, void* cq, int dtype, float eps, int tokens,
                                         int block_size, int num_blocks, int write_kv, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (q_rank < 1 || kv_rank < 1 || rot_dim < 0 || rotary_dim < 0 || rotary_dim > rot_dim || rotary_dim % 2 || !(eps > 0.f) ||
      !x || !wq || !cq)
    return FE_BAD_ARGUMENT;
  if (stride < (long long)q_rank + (write_kv ? kv_rank + rot_dim : 0)) return FE_BAD_ARGUMENT;
  if (write_kv && (!wkv || !key_pages || !positions || !token_seq || !block_table || block_size < 1 || num_blocks < 1 ||
                   (rotary_dim && !inv_freq)))
    return FE_BAD_ARGUMENT;
#define LAUNCH(T)                                                                                                 \
  latent_norm_rope_write_kernel<T><<<tokens, LT_THREADS, 0, stream>>>(                                            \
      x, (size_t)stride, q_rank, kv_rank, rot_dim, rotary_dim, wq, wkv, inv_freq, positions, token_seq, block_table, \
      table_stride, (T*)key_pages, (T*)value_pages, (T*)cq, eps, block_size, num_blocks, write_kv)
  if (dtype == FE_F32) LAUNCH(float);
  else if (dtype == FE_BF16) LAUNCH(bf16_t);
  else return FE_BAD_ARGUMENT;
#undef LAUNCH
  return fe_check_launch();
}

// One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void latent_query_pack_kernel(
    const T* __restrict__ q, size_t q_stride, const T* __restrict__ qa, const float* __restrict__ inv_freq,
    const int* __restrict__ positions, T* __restrict__ out, int tokens, int heads, int dim, int rot_dim, int rotary_dim,
    int kv_rank) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  T* dst = out + ((size_t)t * heads + h) * (kv_rank + rot_dim);
  const T* a = qa + ((size_t)h * tokens + t) * kv_rank;
  for (int c = lane; c < kv_rank; c += 64) dst[c] = a[c];
  const T* r = q + (size_t)t * q_stride + (size_t)h * (dim + rot_dim) + dim;
  const int half = rotary_dim / 2;
  const int pos = positions[t];
  for (int i = lane; i < half; i += 64) {
    float sn, cs;
    sincosf((float)pos * inv_freq[i], &sn, &cs);
    const float u = load_as_float(r + i), v = load_as_float(r + i + half);
    store_from_float(dst + kv_rank + i, u * cs - v * sn);
    store_from_float(dst + kv_rank + i + half, v * cs + u * sn);
  }
  for (int c = rotary_dim + lane; c < rot_dim; c += 64) dst[kv_rank + c] = r[c];
}

extern "C" int fe_latent_query_pack(const void* q, long long q_stride, const void* qa, const float* inv_freq,
                                    const int* positions, void* out, int dtype, int tokens, int heads, int dim,
                                    int rot_dim, int rotary_dim, int kv_rank, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (heads < 1 || heads > 65535 || dim < 1 || kv_rank < 1 || rot_dim < 0 || rotary_dim < 0 || rotary_dim > rot_dim ||
      rotary_dim % 2 || q_stride < (long long)heads * (dim + rot_dim) || !q || !qa || !out || !positions ||
      (rotary_dim && !inv_freq))
    return FE_BAD_ARGUMENT;
  const dim3 grid(tokens, heads);
#define LAUNCH(T)                                                                                          \
  latent_query_pack_kernel<T><<<grid, 64, 0, stream>>>((const T*)q, (size_t)q_stride, (const T*)qa, inv_freq, \
                                                       positions, (T*)out, tokens, heads, dim, rot_dim, rotary_dim, kv_rank)
  if (dtype == FE_F32) LAUNCH(float);
  else if (dtype == FE_BF16) LAUNCH(bf16_t);
  else return FE_BAD_ARGUMENT;
#undef LAUNCH
  return fe_check_launch();
}
