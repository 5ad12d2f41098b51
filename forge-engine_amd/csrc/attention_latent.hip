// Causal attention of many query heads over one shared cache of rows, on the matrix cores (bfloat16).
//
// Every head of a token reads the same cached rows: a row of DK numbers is the key of all heads, and
// its first DV numbers, kept a second time in transposed pages, are the value (attention through a
// latent, after the queries were taken through the keys' up-projection).  Key pages
// [page][1][slot][DK], value pages [page][1][DV][slot]; the step's own rows are already in them.
//
// Block = 4 waves on 64 query rows of one sequence, a row being a (token, head) pair, token-major, so
// that the 64 rows of a block share their keys; a wave owns 16 rows.  Keys are walked in tiles of 32:
// the tile's keys and its transposed values reach LDS by `global_load_lds_dwordx4` (64 lanes x 16 bytes at
// consecutive LDS addresses, no staging registers: every load of a tile is in flight at once), and all
// four waves read their MFMA operands from there.  Which global bytes a lane loads is free, where they
// land is not, so a key row's 16-byte chunks lie permuted by the row's low bits and a value dim's four
// key chunks by the dim's bits 2 and 3: the operand reads of 16 lanes then spread over the banks.  Where two
// blocks fit a CU, one block's loads run under the other's products.  S^T = K Q^T and O^T = V^T P^T on MFMA 16x16x32 with
// scores, statistics and outputs in registers: lane (r = lane % 16, g = lane / 16) holds, of row r,
// the scores of keys 8g .. 8g + 7 of the tile (the key rows of the first product are permuted so that
// they come out that way, which is the order the second product's operands want) and the outputs of
// dims 16t + 4g .. + 3 of every tile t of 16 dims.  Online softmax in base 2, float32.
//
// A launch may cut every block's keys into `splits` runs of whole tiles (grid.y) for steps with few
// rows and long contexts; each run leaves its unnormalised output, maximum and sum in float32, and a
// second kernel merges them in order.  Slots beyond the context may hold anything: their values are
// masked to zero in the operand.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;
typedef __attribute__((ext_vector_type(2))) unsigned int uintx2;

#define LA_KEYS 32
#define LA_ROWS 64

__device__ __forceinline__ unsigned int pack_two(float lo, float hi) {
  return (unsigned int)float_to_bf16(lo) | ((unsigned int)float_to_bf16(hi) << 16);
}

__device__ __forceinline__ void tile_to_lds(const void* global, void* lds) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global,
                                   (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// Queries (DK / 8 registers a lane) and outputs (DV / 4) stay in registers for the whole walk: the sizes that need
// more than half a SIMD's registers for them run one block a CU, the others two.
template <int DK, int DV>
__global__ __launch_bounds__(256, (DK / 8 + DV / 4 > 160) ? 1 : 2) void latent_attention_kernel(
    const bf16_t* __restrict__ q, size_t q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
    const int* __restrict__ block_table, int table_stride, int heads, int block_size, int num_blocks,
    float scale_log2, int splits, int total_rows) {
  constexpr int KC = DK / 32, DT = DV / 16, CHUNKS = DK / 8;
  constexpr int SW = CHUNKS % 8 == 0 ? 7 : (CHUNKS % 4 == 0 ? 3 : 1);     // a key row's chunks are permuted by row & SW
  constexpr int K_UNITS = LA_KEYS * CHUNKS, V_UNITS = DV * 4;             // 16-byte units of a tile's keys and values
  constexpr int LOADS = (K_UNITS + V_UNITS) / 64;                         // load instructions a tile, 64 units each
  static_assert(K_UNITS % 64 == 0 && V_UNITS % 64 == 0, "whole load instructions");
  extern __shared__ __attribute__((aligned(16))) unsigned char tile_lds[];
  const bf16_t* Ks = (const bf16_t*)tile_lds;                             // unit u: key u / CHUNKS, chunk (u % CHUNKS) ^ (key & SW)
  const bf16_t* Vs = (const bf16_t*)(tile_lds + K_UNITS * 16);            // unit u: dim u / 4, keys 8 ((u % 4) ^ (dim >> 2 & 3)) .. + 7

  const int tid = threadIdx.x, lane = tid & 63, lr = lane & 15, lq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int seq = blockIdx.z, split = blockIdx.y;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  const int ctx = ctx_len[seq];
  const int before = ctx - q_len;
  const int rows_total = q_len * heads;
  const int row0 = blockIdx.x * LA_ROWS;
  if (row0 >= rows_total || before < 0) return;

  const int my_row = row0 + wave * 16 + lr;
  const bool row_ok = my_row < rows_total;
  const int tok = row_ok ? my_row / heads : 0;
  const int head = row_ok ? my_row - tok * heads : 0;
  const int pos = before + tok;
  const bool wave_ok = row0 + wave * 16 < rows_total;
  const int wave_pos_max = before + (min(rows_total, row0 + wave * 16 + 16) - 1) / heads;
  const int block_pos_max = before + (min(rows_total, row0 + LA_ROWS) - 1) / heads;
  const int tiles = block_pos_max / LA_KEYS + 1;
  const int run = (tiles + splits - 1) / splits;
  const int t_lo = split * run, t_hi = min(tiles, t_lo + run);

  bf16x8 qb[KC];
  {
    const bf16_t* qrow = q + (size_t)(q0 + tok) * q_stride + (size_t)head * DK + lq * 8;
#pragma unroll
    for (int c = 0; c < KC; ++c)
      qb[c] = row_ok ? *(const bf16x8*)(qrow + c * 32) : __builtin_bit_cast(bf16x8, uintx4{0u, 0u, 0u, 0u});
  }
  floatx4 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const int* table = block_table + (size_t)seq * table_stride;
  const int last_key = ctx - 1;

  for (int tile = t_lo; tile < t_hi; ++tile) {
    const int kb = tile * LA_KEYS;
    __syncthreads();        // the tile before is consumed
    // the wave's share of the tile's loads; keys beyond the context read the last key's page (their scores are
    // masked and their values cleared in the operand), so every address is a valid one
#pragma unroll
    for (int n = 0; n < (LOADS + 3) / 4; ++n) {
      const int load = wave + 4 * n;
      if (load < LOADS) {
        const int u = load * 64 + lane;
        const bf16_t* src;
        if (load < K_UNITS / 64) {
          const int key = u / CHUNKS, slot = u - key * CHUNKS;
          const int kp = min(kb + key, last_key);
          int page = table[kp / block_size];
          page = min(max(page, 0), num_blocks - 1);
          src = key_pages + ((size_t)page * block_size + kp % block_size) * DK + (slot ^ (key & SW)) * 8;
        } else {
          const int uv = u - K_UNITS;
          const int dim = uv >> 2, kc = (uv & 3) ^ ((dim >> 2) & 3);
          const int kp = min(kb + 8 * kc, last_key & ~7);
          int page = table[kp / block_size];
          page = min(max(page, 0), num_blocks - 1);
          src = value_pages + ((size_t)page * DV + dim) * block_size + kp % block_size;
        }
        tile_to_lds(src, tile_lds + load * 1024);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (!wave_ok || kb > wave_pos_max) continue;      // the whole wave: no row, or no row that sees this tile

    floatx4 st[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      st[h] = floatx4{0.f, 0.f, 0.f, 0.f};
      // operand row lr of half h is key 8 (lr / 4) + 4 h + lr % 4, so that result row 4 g + i is key 8 g + 4 h + i
      const int key = 8 * (lr >> 2) + 4 * h + (lr & 3);
      const bf16_t* krow = Ks + (size_t)key * DK;
#pragma unroll
      for (int c = 0; c < KC; ++c)
        st[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(krow + ((c * 4 + lq) ^ (key & SW)) * 8), qb[c], st[h], 0, 0, 0);
    }
    float s[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = kb + 8 * lq + j;
      s[j] = (row_ok && key <= pos) ? st[j >> 2][j & 3] * scale_log2 : -INFINITY;
      mx = fmaxf(mx, s[j]);
    }
    mx = max_xor32(max_xor16(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new > -INFINITY ? m_new : 0.f;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s[j] = __builtin_amdgcn_exp2f(s[j] - m_use);
      sum += s[j];
    }
    sum = sum_xor32(sum_xor16(sum));
    l_run = l_run * corr + sum;
    m_run = m_new;
    const bf16x8 pb = __builtin_bit_cast(bf16x8, uintx4{pack_two(s[0], s[1]), pack_two(s[2], s[3]), pack_two(s[4], s[5]), pack_two(s[6], s[7])});

    // this lane's eight keys of the value operand: those beyond the context are cleared
    const int vkey = kb + 8 * lq;
    uintx4 v_mask;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const unsigned int lo = vkey + 2 * w < ctx ? 0x0000ffffu : 0u;
      const unsigned int hi = vkey + 2 * w + 1 < ctx ? 0xffff0000u : 0u;
      v_mask[w] = lo | hi;
    }
    const bf16_t* vrow = Vs + ((size_t)lr * 4 + (lq ^ ((lr >> 2) & 3))) * 8;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      const uintx4 va = *(const uintx4*)(vrow + (size_t)t * 16 * 32) & v_mask;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] *= corr;
      o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, va), pb, o[t], 0, 0, 0);
    }
  }

  if (!row_ok) return;
  const size_t global_row = (size_t)(q0 + tok) * heads + head;
  if (splits == 1) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    bf16_t* orow = out + global_row * DV + 4 * lq;
#pragma unroll
    for (int t = 0; t < DT; ++t)
      *(uintx2*)(orow + 16 * t) = uintx2{pack_two(o[t][0] * inv, o[t][1] * inv), pack_two(o[t][2] * inv, o[t][3] * inv)};
    return;
  }
  float* po = part_o + ((size_t)split * total_rows + global_row) * DV + 4 * lq;
#pragma unroll
  for (int t = 0; t < DT; ++t) *(floatx4*)(po + 16 * t) = o[t];
  if (lq == 0) {
    float* pm = part_ml + ((size_t)split * total_rows + global_row) * 2;
    pm[0] = m_run;
    pm[1] = l_run;
  }
}

// out[row] = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m), m the largest m_s; the runs in order.
__global__ __launch_bounds__(128) void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                           bf16_t* __restrict__ out, int splits, int total_rows, int dv) {
  const int row = blockIdx.x;
  float top = -INFINITY;
  for (int s = 0; s < splits; ++s) top = fmaxf(top, part_ml[((size_t)s * total_rows + row) * 2]);
  const float m_use = top > -INFINITY ? top : 0.f;
  float denom = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float* pm = part_ml + ((size_t)s * total_rows + row) * 2;
    denom += pm[1] * __builtin_amdgcn_exp2f(pm[0] - m_use);
  }
  const float inv = denom > 0.f ? 1.f / denom : 0.f;
  for (int d = threadIdx.x; d < dv; d += 128) {
    float acc = 0.f;
    for (int s = 0; s < splits; ++s) {
      const size_t at = (size_t)s * total_rows + row;
      acc += part_o[at * dv + d] * __builtin_amdgcn_exp2f(part_ml[at * 2] - m_use);
    }
    out[(size_t)row * dv + d] = float_to_bf16(acc * inv);
  }
}

template <int DK, int DV>
static int launch_latent(const void* q, long long q_stride, const void* key_pages, const void* value_pages, void* out,
                         float* part_o, float* part_ml, const int* cu_q, const int* ctx_len, const int* block_table,
                         int table_stride, int num_seqs, int max_q_len, int heads, int block_size, int num_blocks,
                         float scale, int splits, int tokens, hipStream_t stream) {
  const long long rows = (long long)max_q_len * heads;
  const dim3 grid((unsigned)((rows + LA_ROWS - 1) / LA_ROWS), splits, num_seqs);
  constexpr int lds = (LA_KEYS * DK + DV * 32) * 2;       // a tile's keys and its transposed values
  static bool sized = false;                              // more than 64 KB of LDS a block has to be asked for, once a kernel
  if (lds > 64 * 1024 && !sized) {
    if (hipFuncSetAttribute((const void*)latent_attention_kernel<DK, DV>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return FE_LAUNCH_FAILED;
    sized = true;
  }
  latent_attention_kernel<DK, DV><<<grid, 256, lds, stream>>>(
      (const bf16_t*)q, (size_t)q_stride, (const bf16_t*)key_pages, (const bf16_t*)value_pages, (bf16_t*)out, part_o,
      part_ml, cu_q, ctx_len, block_table, table_stride, heads, block_size, num_blocks, scale * 1.4426950408889634f,
      splits, tokens * heads);
  if (splits > 1) latent_merge_kernel<<<tokens * heads, 128, 0, stream>>>(part_o, part_ml, (bf16_t*)out, splits, tokens * heads, DV);
  return fe_check_launch();
}

// The (DK, DV) pairs compiled below; 0 for any other.
extern "C" int fe_latent_attention_supported(int row_dim, int value_dim) {
  return (row_dim == 576 && value_dim == 512) || (row_dim == 320 && value_dim == 256) || (row_dim == 192 && value_dim == 128) ||
         (row_dim == 128 && value_dim == 96) || (row_dim == 96 && value_dim == 64);
}

extern "C" int fe_latent_attention(const void* q, long long q_stride, const void* key_pages, const void* value_pages, void* out,
                                   float* part_o, float* part_ml, const int* cu_q, const int* ctx_len,
                                   const int* block_table, int table_stride, int num_seqs, int max_q_len, int heads,
                                   int row_dim, int value_dim, int block_size, int num_blocks, float scale, int splits,
                                   int tokens, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (heads < 1 || max_q_len < 1 || block_size < 8 || block_size % 8 || num_blocks < 1 || splits < 1 || splits > 64 ||
      num_seqs > 65535 || q_stride < (long long)heads * row_dim || q_stride % 8 || (splits > 1 && (!part_o || !part_ml)) ||
      (long long)tokens * heads > 0x7fffffffLL || !fe_latent_attention_supported(row_dim, value_dim))
    return FE_BAD_ARGUMENT;
#define CASE(DK, DV)                                                                                                   \
  if (row_dim == DK && value_dim == DV)                                                                                \
    return launch_latent<DK, DV>(q, q_stride, key_pages, value_pages, out, part_o, part_ml, cu_q, ctx_len, block_table, \
                                 table_stride, num_seqs, max_q_len, heads, block_size, num_blocks, scale, splits, tokens, stream)
  CASE(576, 512);
  CASE(320, 256);
  CASE(192, 128);
  CASE(128, 96);
  CASE(96, 64);
#undef CASE
  return FE_BAD_ARGUMENT;
}
