// Paged grouped-query attention for a mixed batch with the masks and softmax forms beyond the plain
// causal one, on the vector ALU in float32:
//   * the query at position p reads keys j <= p with j > p - window (window > 0) and
//     j >= p - p % chunk (chunk > 0: runs of `chunk` positions counted from position 0);
//   * a sink per query head: exp(sink_h) joins the softmax's denominator, with no key and no value
//     (the running maximum starts at sink_h and the running sum at 1);
//   * values of another width than keys;
//   * an output gate: the result times sigmoid(gate), a gate per element or one per query head;
//   * a soft cap: scores, after the scale, become cap * tanh(score / cap);
//   * a penalty on distance: slope_h * (p - j) comes off head h's score of key j (after scale and cap);
//   * a bias by distance: table[h][min(p - j, span - 1)] is added to head h's score of key j (after the scale,
//     which does not multiply it); the table is float32 [heads][span];
//   * keys that are their own values (no value pages): a key's first Dv dims are read as its value.
// One launch serves portions of prompts and single tokens alike; the step's own keys and values are
// already in the pages (keys [page][kv head][slot][D], values transposed [page][kv head][Dv][slot]).
// Block = (tile of 16 rows, kv head, sequence), a row being a (query token, head of the group) pair,
// so that the heads sharing a kv head share its tiles.  Thread (r = tid / 16, c = tid % 16) owns row
// r: scores of keys c, c + 16 of a tile and output dims c, c + 16, ...; a row's 16 lanes meet by
// shuffles.  Online softmax over key tiles; one rounding at the store.
#include "common.h"

#define ROWS 16

template <typename T, int TK, int DPT>
__global__ __launch_bounds__(256) void masked_attention_kernel(
    const T* __restrict__ q, size_t q_stride, const T* __restrict__ key_pages, const T* __restrict__ value_pages,
    T* __restrict__ out, const T* __restrict__ gate, size_t gate_stride, const float* __restrict__ sink,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int table_stride, int kv_heads, int groups, int D, int Dv, int block_size, int num_blocks, int window,
    int chunk, float scale, float softcap, int head_gate, const float* __restrict__ slopes,
    const float* __restrict__ dist_bias, int span) {
  constexpr int KPT = TK / 16;
  extern __shared__ float smem[];
  const int ks = D + 1, vs = Dv + 1;
  float* Qs = smem;                 // [ROWS][D + 1]
  float* Ks = Qs + ROWS * ks;       // [TK][D + 1]
  float* Vs = Ks + TK * ks;         // [TK][Dv + 1]
  float* Ps = Vs + (value_pages ? TK * vs : 0);   // [ROWS][TK]; keys that are their own values keep no value tile

  const int seq = blockIdx.z, hk = blockIdx.y;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  const int ctx = ctx_len[seq];
  const int before = ctx - q_len;
  const int rows_total = q_len * groups;
  const int row0 = blockIdx.x * ROWS;
  if (row0 >= rows_total || before < 0) return;

  const int tid = threadIdx.x, r = tid / 16, c = tid % 16;
  const int my_row = row0 + r;
  const bool row_ok = my_row < rows_total;
  const int my_tok = row_ok ? my_row / groups : 0;
  const int my_g = row_ok ? my_row - my_tok * groups : 0;
  const int my_pos = before + my_tok;
  auto first_seen = [&](int p) {
    int f = window > 0 ? max(0, p - window + 1) : 0;
    if (chunk > 0) f = max(f, p / chunk * chunk);
    return f;
  };
  const int my_first = first_seen(my_pos);
  const int last_row = min(rows_total, row0 + ROWS) - 1;
  const int pos_min = before + row0 / groups, pos_max = before + last_row / groups;
  // the first key any row of the tile reads: positions rise with the rows, but a run's start does
  // not fall, so the tile's first row has the smallest
  const int k_begin = first_seen(pos_min), k_end = pos_max + 1;

  for (int e = tid; e < ROWS * D; e += 256) {
    const int rr = e / D, d = e - rr * D;
    const int row = row0 + rr;
    float v = 0.f;
    if (row < rows_total) {
      const int tok = row / groups, g = row - tok * groups;
      v = load_as_float(q + (size_t)(q0 + tok) * q_stride + (size_t)(hk * groups + g) * D + d);
    }
    Qs[rr * ks + d] = v;
  }

  const int head = hk * groups + my_g;
  const float slope = slopes ? slopes[head] : 0.f;
  const float* bias_row = dist_bias ? dist_bias + (size_t)head * span : nullptr;
  float m = sink ? sink[head] : -INFINITY;
  float l = sink ? 1.f : 0.f;
  float acc[DPT];
#pragma unroll
  for (int i = 0; i < DPT; ++i) acc[i] = 0.f;
  const int* table = block_table + (size_t)seq * table_stride;

  for (int kt = k_begin / TK * TK; kt < k_end; kt += TK) {
    __syncthreads();   // the tile before is consumed; Q is visible on the first pass
    for (int e = tid; e < TK * D; e += 256) {
      const int kk = e / D, d = e - kk * D;
      const int kp = kt + kk;
      float v = 0.f;
      if (kp >= k_begin && kp < k_end) {
        const int page = table[kp / block_size];
        if (page >= 0 && page < num_blocks)
          v = load_as_float(key_pages + (((size_t)page * kv_heads + hk) * block_size + kp % block_size) * D + d);
      }
      Ks[kk * ks + d] = v;
    }
    for (int e = tid; value_pages && e < TK * Dv; e += 256) {
      const int d = e / TK, kk = e - d * TK;
      const int kp = kt + kk;
      float v = 0.f;
      if (kp >= k_begin && kp < k_end) {
        const int page = table[kp / block_size];
        if (page >= 0 && page < num_blocks)
          v = load_as_float(value_pages + (((size_t)page * kv_heads + hk) * Dv + d) * block_size + kp % block_size);
      }
      Vs[kk * vs + d] = v;
    }
    __syncthreads();

    float s[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) s[i] = 0.f;
    const float* qrow = Qs + r * ks;
    for (int d = 0; d < D; ++d) {
      const float qv = qrow[d];
#pragma unroll
      for (int i = 0; i < KPT; ++i) s[i] = fmaf(qv, Ks[(c + 16 * i) * ks + d], s[i]);
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int kp = kt + c + 16 * i;
      const bool visible = row_ok && kp <= my_pos && kp >= my_first;
      float score = s[i] * scale;
      if (softcap > 0.f) score = softcap * tanhf(score / softcap);
      if (slopes) score -= slope * (float)(my_pos - kp);
      if (bias_row && visible) score += bias_row[min(my_pos - kp, span - 1)];
      s[i] = visible ? score : -INFINITY;
      tile_max = fmaxf(tile_max, s[i]);
    }
#pragma unroll
    for (int offset = 8; offset > 0; offset >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, offset, FE_WAVE));
    const float m_new = fmaxf(m, tile_max);
    float corr = 1.f, tile_sum = 0.f;
    if (m_new > -INFINITY) {
      corr = expf(m - m_new);
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        s[i] = expf(s[i] - m_new);
        tile_sum += s[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < KPT; ++i) s[i] = 0.f;
    }
#pragma unroll
    for (int offset = 8; offset > 0; offset >>= 1) tile_sum += __shfl_xor(tile_sum, offset, FE_WAVE);
    l = l * corr + tile_sum;
    m = m_new;
#pragma unroll
    for (int i = 0; i < KPT; ++i) Ps[r * TK + c + 16 * i] = s[i];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < DPT; ++i) acc[i] *= corr;
    const float* prow = Ps + r * TK;
    for (int kk = 0; kk < TK; ++kk) {
      const float p = prow[kk];
      const float* vrow = value_pages ? Vs + kk * vs : Ks + kk * ks;
#pragma unroll
      for (int i = 0; i < DPT; ++i)
        if (c + 16 * i < Dv) acc[i] = fmaf(p, vrow[c + 16 * i], acc[i]);
    }
  }

  if (row_ok) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const size_t at = (size_t)head * Dv;
    T* orow = out + (size_t)(q0 + my_tok) * ((size_t)kv_heads * groups * Dv) + at;
    const T* grow = gate ? gate + (size_t)(q0 + my_tok) * gate_stride + (head_gate ? (size_t)head : at) : nullptr;
    const float whole = (grow && head_gate) ? 1.f / (1.f + expf(-load_as_float(grow))) : 1.f;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int d = c + 16 * i;
      if (d < Dv) {
        float v = acc[i] * inv * whole;
        if (grow && !head_gate) v *= 1.f / (1.f + expf(-load_as_float(grow + d)));
        store_from_float(orow + d, v);
      }
    }
  }
}

template <typename T>
static int launch_masked(const void* q, long long q_stride, const void* key_pages, const void* value_pages, void* out,
                         const void* gate, long long gate_stride, const float* sink, const int* cu_q,
                         const int* ctx_len, const int* block_table, int table_stride, int num_seqs, int max_q_len,
                         int q_heads, int kv_heads, int D, int Dv, int block_size, int num_blocks, int window,
                         int chunk, float scale, float softcap, int head_gate, const float* slopes, const float* dist_bias,
                         int span, hipStream_t stream) {
  const int groups = q_heads / kv_heads;
  const long long rows = (long long)max_q_len * groups;
  const dim3 grid((unsigned)((rows + ROWS - 1) / ROWS), kv_heads, num_seqs);
  const int held = value_pages ? Dv + 1 : 0;      // values that are the keys' own dims need no tile of their own
  const int tk = D + held <= 256 ? 32 : 16;
  const size_t lds = ((size_t)ROWS * (D + 1) + (size_t)tk * (D + 1) + (size_t)tk * held + (size_t)ROWS * tk) * sizeof(float);
#define LAUNCH(TK, DPT)                                                                                          \
  do {                                                                                                           \
    if (lds > 64 * 1024 &&                                                                                       \
        hipFuncSetAttribute((const void*)masked_attention_kernel<T, TK, DPT>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                            (int)lds) != hipSuccess)                                                             \
      return FE_BAD_ARGUMENT;                                                                                    \
    masked_attention_kernel<T, TK, DPT><<<grid, 256, lds, stream>>>(                                             \
        (const T*)q, (size_t)q_stride, (const T*)key_pages, (const T*)value_pages, (T*)out, (const T*)gate,      \
        (size_t)gate_stride, sink, cu_q, ctx_len, block_table, table_stride, kv_heads, groups, D, Dv, block_size, \
        num_blocks, window, chunk, scale, softcap, head_gate, slopes, dist_bias, span);                          \
  } while (0)
  if (lds > 150 * 1024) return FE_BAD_ARGUMENT;
  if (tk == 32) {
    if (Dv <= 64) LAUNCH(32, 4);
    else if (Dv <= 128) LAUNCH(32, 8);
    else if (Dv <= 256) LAUNCH(32, 16);
    else LAUNCH(32, 32);
  } else {
    if (Dv <= 64) LAUNCH(16, 4);
    else if (Dv <= 128) LAUNCH(16, 8);
    else if (Dv <= 256) LAUNCH(16, 16);
    else LAUNCH(16, 32);
  }
#undef LAUNCH
  return fe_check_launch();
}

extern "C" int fe_masked_attention(const void* q, int dtype, long long q_stride, const void* key_pages,
                                   const void* value_pages, void* out, const void* gate, long long gate_stride,
                                   const float* sink, const int* cu_q, const int* ctx_len, const int* block_table,
                                   int table_stride, int num_seqs, int max_q_len, int q_heads, int kv_heads,
                                   int head_dim, int value_dim, int block_size, int num_blocks, int window, int chunk,
                                   float scale, float softcap, int head_gate, int tokens, const float* slopes,
                                   const float* dist_bias, int span, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads || head_dim < 1 || head_dim > 640 || value_dim < 1 ||
      value_dim > 512 || (!value_pages && value_dim > head_dim) || (dist_bias && span < 1) || block_size <= 0 || num_blocks <= 0 || max_q_len < 1 || window < 0 || chunk < 0 ||
      num_seqs > 65535 || kv_heads > 65535)
    return FE_BAD_ARGUMENT;
  if (q_stride < (long long)q_heads * head_dim || softcap < 0.f ||
      (gate && gate_stride < (long long)q_heads * (head_gate ? 1 : value_dim)))
    return FE_BAD_ARGUMENT;
  if (dtype == FE_F32)
    return launch_masked<float>(q, q_stride, key_pages, value_pages, out, gate, gate_stride, sink, cu_q, ctx_len,
                                block_table, table_stride, num_seqs, max_q_len, q_heads, kv_heads, head_dim, value_dim,
                                block_size, num_blocks, window, chunk, scale, softcap, head_gate, slopes, dist_bias, span, stream);
  if (dtype == FE_BF16)
    return launch_masked<bf16_t>(q, q_stride, key_pages, value_pages, out, gate, gate_stride, sink, cu_q, ctx_len,
                                 block_table, table_stride, num_seqs, max_q_len, q_heads, kv_heads, head_dim, value_dim,
                                 block_size, num_blocks, window, chunk, scale, softcap, head_gate, slopes, dist_bias, span, stream);
  return FE_BAD_ARGUMENT;
}
