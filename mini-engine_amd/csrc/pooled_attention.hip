// What attention over a sliding window with pooled blocks needs before its scores: the queries and keys normed over their
// whole projection, the page writes, and the means of whole blocks of keys and values.
//
//   scatter   a block a token: q (all heads' nh * d elements at once) and k (nkv * d) are each divided by the root mean square
//             of the whole row and multiplied by a weight of the row's size; the normed keys go to the key pages. The values
//             are the keys as projected (before the norm) when no column of values is given, else that column's nkv * dv
//             elements; they go to the value pages (transposed).
//   pool      block b of an item holds the positions b P .. b P + P - 1. The token at position b P + P - 1 completes it: for
//             every token of the step that completes a block, the mean of the block's P keys as the pages hold them and the
//             mean of its P values are written to the pooled pages, at entry b: page table[b / bs], slot b % bs, the same
//             layouts as the pages of tokens. A block may have begun in an earlier step: its keys are read from the pages.
//             The sum runs in ascending position, so a block's mean does not depend on how the sequence was cut.
//
// Layouts: keys K[page, kv_head, slot, d]; values transposed V[page, kv_head, dv, slot]; pooled pages alike.
#include "common.h"

#define WN_Q_HELD 16
#define WN_K_HELD 8
template <typename T>
__global__ __launch_bounds__(256) void whole_norm_scatter_kernel(
    const T* __restrict__ proj, long long row, int c_q, int c_k, int c_v, const float* __restrict__ q_w, const float* __restrict__ k_w,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table, int table_width,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int nh, int nkv, int d, int dv, int bs, float eps,
    T* __restrict__ k_pool, T* __restrict__ v_pool, int own_pool) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const T* p = proj + (size_t)t * row;
  const int nq = nh * d, nk = nkv * d;
  // (asked for ahead of the sums: the page's number is two trips to memory away)
  const int pos = positions[t];
  const int page = block_table[(size_t)token_item[t] * table_width + pos / bs], slot = pos % bs;
  if (nq <= WN_Q_HELD * 256 && nk <= WN_K_HELD * 256 && (c_v < 0 || dv == d)) {
    // Rows that the block's registers hold (queries of up to 4,096 elements, keys of up to 2,048): the row and the weights are
    // asked for once, together, and the block waits for memory twice (loads, then the two sums as one exchange), not five times.
    float qv[WN_Q_HELD], qw[WN_Q_HELD], kv[WN_K_HELD], kw[WN_K_HELD], vv[WN_K_HELD];
    float sq = 0.f, sk = 0.f;
#pragma unroll
    for (int n = 0; n < WN_Q_HELD; ++n) {
      const int i = threadIdx.x + 256 * n;
      qv[n] = i < nq ? to_float(p[c_q + i]) : 0.f;
      qw[n] = i < nq ? q_w[i] : 0.f;
    }
#pragma unroll
    for (int n = 0; n < WN_K_HELD; ++n) {
      const int i = threadIdx.x + 256 * n;
      kv[n] = i < nk ? to_float(p[c_k + i]) : 0.f;
      kw[n] = i < nk ? k_w[i] : 0.f;
      vv[n] = c_v >= 0 && i < nk ? to_float(p[c_v + i]) : kv[n];  // the values: a column of their own, or the keys as projected
    }
#pragma unroll
    for (int n = 0; n < WN_Q_HELD; ++n) sq = fmaf(qv[n], qv[n], sq);
#pragma unroll
    for (int n = 0; n < WN_K_HELD; ++n) sk = fmaf(kv[n], kv[n], sk);
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    const int lane = threadIdx.x & (ME_WAVE - 1), wave = threadIdx.x / ME_WAVE;
    if (lane == 0) {
      red[wave] = sq;
      red[4 + wave] = sk;
    }
    __syncthreads();
    const float rq = rsqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)nq + eps);
    const float rk = rsqrtf(((red[4] + red[5]) + (red[6] + red[7])) / (float)nk + eps);
    T* qo = q_out + (size_t)t * nq;
#pragma unroll
    for (int n = 0; n < WN_Q_HELD; ++n) {
      const int i = threadIdx.x + 256 * n;
      if (i < nq) qo[i] = from_float<T>(qv[n] * rq * qw[n]);
    }
#pragma unroll
    for (int n = 0; n < WN_K_HELD; ++n) {
      const int i = threadIdx.x + 256 * n;
      if (i < nk) {
        const int kvh = i / d, e = i % d;
        const T key = from_float<T>(kv[n] * rk * kw[n]), value = from_float<T>(vv[n]);
        k_cache[(((size_t)page * nkv + kvh) * bs + slot) * d + e] = key;
        v_cache[(((size_t)page * nkv + kvh) * dv + e) * bs + slot] = value;
        if (own_pool > 0 && (pos + 1) % own_pool == 0) {
          // A step of single tokens (the host says so): the token that completes a pooled block adds up the block itself. The
          // block's earlier keys came in earlier steps and lie in the pages; its own key is the last and is added last, as
          // rounded: the sums are those of pool_blocks_kernel, in its order, and the launch of that kernel is saved.
          const int b = pos / own_pool, first = b * own_pool;
          const int* table = block_table + (size_t)token_item[t] * table_width;
          float ks = 0.f, vs = 0.f;
#pragma unroll 8
          for (int j = 0; j < own_pool - 1; ++j) {
            const int at = first + j, pg = table[at / bs], sl = at % bs;
            ks += to_float(k_cache[(((size_t)pg * nkv + kvh) * bs + sl) * d + e]);
            vs += to_float(v_cache[(((size_t)pg * nkv + kvh) * dv + e) * bs + sl]);
          }
          ks += to_float(key);
          vs += to_float(value);
          const int to_page = table[b / bs], to_slot = b % bs;
          const float share = 1.f / (float)own_pool;
          k_pool[(((size_t)to_page * nkv + kvh) * bs + to_slot) * d + e] = from_float<T>(ks * share);
          v_pool[(((size_t)to_page * nkv + kvh) * dv + e) * bs + to_slot] = from_float<T>(vs * share);
        }
      }
    }
    return;
  }
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const float x = to_float(p[c_q + i]);
    sq = fmaf(x, x, sq);
  }
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const float x = to_float(p[c_k + i]);
    sk = fmaf(x, x, sk);
  }
  const float rq = rsqrtf(block_sum(sq, red) / (float)nq + eps);
  const float rk = rsqrtf(block_sum(sk, red) / (float)nk + eps);
  T* qo = q_out + (size_t)t * nq;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) qo[i] = from_float<T>(to_float(p[c_q + i]) * rq * q_w[i]);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int kvh = i / d, e = i % d;
    k_cache[(((size_t)page * nkv + kvh) * bs + slot) * d + e] = from_float<T>(to_float(p[c_k + i]) * rk * k_w[i]);
  }
  const int vcol = c_v >= 0 ? c_v : c_k;  // the values: a column of their own, or the keys as projected
  for (int i = threadIdx.x; i < nkv * dv; i += blockDim.x) {
    const int kvh = i / dv, e = i % dv;
    v_cache[(((size_t)page * nkv + kvh) * dv + e) * bs + slot] = p[vcol + i];
  }
}

// Grid (runs of POOL_TOKENS tokens, kv heads), 256 threads: a block looks at its tokens one after the other and skips those that
// complete no pooled block (a block of the grid for every token cost a step of 2,048 tokens more in starting blocks that had
// nothing to do than in the work). For the others it fetches the pooled block's keys and values 16 positions at a time into
// LDS ((d + dv) * 64 bytes), all loads of a round on their way together, and adds them up there, a thread an element, in
// ascending position.
#define POOL_TOKENS 8
#define POOL_ROUND 16
#define POOL_MAX_ROW 512  // d + dv at most
template <typename T>
__global__ __launch_bounds__(256) void pool_blocks_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                          T* __restrict__ k_pool, T* __restrict__ v_pool,
                                                          const int* __restrict__ positions, const int* __restrict__ token_item,
                                                          const int* __restrict__ block_table, int table_width, int nkv, int d, int dv,
                                                          int bs, int pool, int num_tokens) {
  extern __shared__ float tile[];  // [POOL_ROUND][d + dv]
  const int kvh = blockIdx.y, tid = threadIdx.x;
  for (int t = blockIdx.x * POOL_TOKENS; t < min(num_tokens, (int)(blockIdx.x + 1) * POOL_TOKENS); ++t) {
  const int pos = positions[t];
  if ((pos + 1) % pool) continue;  // (the same for every thread of the block)
  const int b = pos / pool, first = b * pool, w = d + dv;
  const int* table = block_table + (size_t)token_item[t] * table_width;
  float sum[POOL_MAX_ROW / 256] = {0.f, 0.f};
  for (int j0 = 0; j0 < pool; j0 += POOL_ROUND) {
    const int n = min(POOL_ROUND, pool - j0);
    for (int i = tid; i < n * d; i += 256) {  // neighbouring threads: neighbouring elements of a key
      const int j = i / d, e = i % d, key = first + j0 + j;
      tile[j * w + e] = to_float(k_cache[(((size_t)table[key / bs] * nkv + kvh) * bs + key % bs) * d + e]);
    }
    for (int i = tid; i < n * dv; i += 256) {  // neighbouring threads: neighbouring slots of a value's element
      const int ev = i / n, j = i % n, key = first + j0 + j;
      tile[j * w + d + ev] = to_float(v_cache[(((size_t)table[key / bs] * nkv + kvh) * dv + ev) * bs + key % bs]);
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < POOL_MAX_ROW / 256; ++q) {
      const int e = tid + 256 * q;
      if (e < w)
        for (int j = 0; j < n; ++j) sum[q] += tile[j * w + e];
    }
    __syncthreads();
  }
  const int to_page = table[b / bs], to_slot = b % bs;
  const float inv = 1.f / (float)pool;
#pragma unroll
  for (int q = 0; q < POOL_MAX_ROW / 256; ++q) {
    const int e = tid + 256 * q;
    if (e < d)
      k_pool[(((size_t)to_page * nkv + kvh) * bs + to_slot) * d + e] = from_float<T>(sum[q] * inv);
    else if (e < w)
      v_pool[(((size_t)to_page * nkv + kvh) * dv + (e - d)) * bs + to_slot] = from_float<T>(sum[q] * inv);
  }
  }
}

// proj [T, row]: queries at column c_q (nh * d), keys at c_k (nkv * d), values at c_v (nkv * dv; c_v < 0: the values are the
// keys as projected, dv == d). q_w float32 [nh * d], k_w float32 [nkv * d]. pool > 0: the pooled pages get the blocks that
// the step's tokens complete.
extern "C" int me_whole_norm_scatter_step(const void* proj, long long row, int c_q, int c_k, int c_v, const float* q_w, const float* k_w,
                                          const int* positions, const int* token_item, const int* block_table, int table_width,
                                          void* q_out, void* k_cache, void* v_cache, void* k_pool, void* v_pool, int num_tokens, int nh,
                                          int nkv, int d, int dv, int bs, int pool, float eps, int single_tokens, int dtype,
                                          hipStream_t stream);

extern "C" int me_whole_norm_scatter(const void* proj, long long row, int c_q, int c_k, int c_v, const float* q_w, const float* k_w,
                                     const int* positions, const int* token_item, const int* block_table, int table_width,
                                     void* q_out, void* k_cache, void* v_cache, void* k_pool, void* v_pool, int num_tokens, int nh,
                                     int nkv, int d, int dv, int bs, int pool, float eps, int dtype, hipStream_t stream) {
  return me_whole_norm_scatter_step(proj, row, c_q, c_k, c_v, q_w, k_w, positions, token_item, block_table, table_width, q_out, k_cache,
                                    v_cache, k_pool, v_pool, num_tokens, nh, nkv, d, dv, bs, pool, eps, 0, dtype, stream);
}

// As me_whole_norm_scatter; single_tokens != 0: every item of the step brings one token (every earlier position of a pooled block
// then lies in the pages already), and the kernel that writes the pages adds up the pooled blocks itself where it holds the rows
// in registers.
extern "C" int me_whole_norm_scatter_step(const void* proj, long long row, int c_q, int c_k, int c_v, const float* q_w, const float* k_w,
                                          const int* positions, const int* token_item, const int* block_table, int table_width,
                                          void* q_out, void* k_cache, void* v_cache, void* k_pool, void* v_pool, int num_tokens, int nh,
                                          int nkv, int d, int dv, int bs, int pool, float eps, int single_tokens, int dtype,
                                          hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (nh <= 0 || nkv <= 0 || nkv > 65535 || d <= 0 || dv <= 0 || bs <= 0 || table_width <= 0 || pool < 0)
    return me_fail("me_whole_norm_scatter: nh=%d nkv=%d d=%d dv=%d bs=%d pool=%d", nh, nkv, d, dv, bs, pool);
  if (c_v < 0 && dv != d) return me_fail("me_whole_norm_scatter: values that are the keys have the keys' size, not %d", dv);
  if (c_q < 0 || c_q + (long long)nh * d > row || c_k < 0 || c_k + (long long)nkv * d > row ||
      (c_v >= 0 && c_v + (long long)nkv * dv > row))
    return me_fail("me_whole_norm_scatter: columns %d, %d, %d of a row of %lld", c_q, c_k, c_v, row);
  if (pool > 0 && (!k_pool || !v_pool)) return me_fail("me_whole_norm_scatter: pooled blocks need pages of their own");
  if (pool > 0 && d + dv > POOL_MAX_ROW) return me_fail("me_whole_norm_scatter: pooled keys and values of %d + %d elements (at most %d)", d, dv, POOL_MAX_ROW);
  // (the rows that the page-write kernel holds in registers: see its first branch)
  const bool own_pool = single_tokens && pool > 0 && (long long)nh * d <= WN_Q_HELD * 256 && (long long)nkv * d <= WN_K_HELD * 256 &&
                        (c_v < 0 || dv == d);
#define WN_RUN(TT)                                                                                                                \
  do {                                                                                                                            \
    whole_norm_scatter_kernel<TT><<<num_tokens, 256, 0, stream>>>((const TT*)proj, row, c_q, c_k, c_v, q_w, k_w, positions,        \
                                                                  token_item, block_table, table_width, (TT*)q_out, (TT*)k_cache, \
                                                                  (TT*)v_cache, nh, nkv, d, dv, bs, eps, (TT*)k_pool,             \
                                                                  (TT*)v_pool, own_pool ? pool : 0);                              \
    if (pool > 0 && !own_pool)                                                                                                    \
      pool_blocks_kernel<TT><<<dim3((num_tokens + POOL_TOKENS - 1) / POOL_TOKENS, nkv), 256,                                       \
                               (size_t)POOL_ROUND * (d + dv) * sizeof(float), stream>>>(                                          \
          (const TT*)k_cache, (const TT*)v_cache, (TT*)k_pool, (TT*)v_pool, positions, token_item, block_table, table_width, nkv, \
          d, dv, bs, pool, num_tokens);                                                                                                       \
  } while (0)
  if (dtype == ME_F32)
    WN_RUN(float);
  else
    WN_RUN(bf16_t);
#undef WN_RUN
  return me_check_launch("me_whole_norm_scatter");
}
