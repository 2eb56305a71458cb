// What attention whose q and k are normed over their whole projection needs before its scores, in its general form: a short
// causal convolution over time on every channel of q, k and v, the norm, a rotation by the position, and the page writes.
//
//   scatter   a block a token. Channel c of [q | k | v] becomes y_t[c] = sum_j w[c, j] * u_(t - taps + 1 + j)[c], where u are
//             the projections as the product left them: those of the step's own tokens lie in the step's memory, the taps - 1
//             before an item's first token in the item's state row (zeros before position 0). q (all heads at once) and k are
//             divided by the root mean square of their whole row and multiplied by a weight of the row's size; then the first
//             `rotary` elements of every head of q and k are turned by the position's angles (element i with i + rotary/2).
//             The queries go to q_out, keys and values to the pages. taps == 0: no convolution. rotary == 0: no rotation.
//   keep      an item's state row afterwards: the last taps - 1 projections of the sequence, oldest first. It runs as a launch
//             of its own behind the scatter, which still reads the rows as the step before left them.
//
// Layouts: keys K[page, kv_head, slot, d]; values transposed V[page, kv_head, dv, slot]; conv weights float32 [nq + nk + nv,
// taps]; state float32 [slots, taps - 1, nq + nk + nv]; rotary table float32 [positions, 2, rotary/2] (cosines, then sines).
#include "common.h"

// TMAX: the most taps this instance takes (its loops over taps are unrolled to that many, so that all of a thread's loads, of four
// channels at a time, are on their way together: a step of single tokens waits for memory once, not once per channel and tap).
template <typename T, int TMAX>
__global__ __launch_bounds__(1024) void conv_norm_rope_scatter_kernel(
    const T* __restrict__ proj, long long row, int c_q, int c_k, int c_v, const float* __restrict__ conv_w, int taps,
    const float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ item_start,
    const float* __restrict__ q_w, const float* __restrict__ k_w, const float* __restrict__ rope, int rotary,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table, int table_width,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int nh, int nkv, int d, int dv, int bs, float eps) {
  extern __shared__ float vals[];  // [nq + nk + nv]: the token's q, k and v behind the convolution, then behind the norm
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int nq = nh * d, nk = nkv * d, nv = nkv * dv, C = nq + nk + nv;
  const int item = token_item[t], pos = positions[t];
  const int first = item_start[item];
  const int page = block_table[(size_t)item * table_width + pos / bs], slot = pos % bs;
  const float* srow = taps > 1 ? state + (size_t)state_slots[item] * (taps - 1) * C : nullptr;
  auto column = [&](int c) { return c < nq ? c_q + c : (c < nq + nk ? c_k + (c - nq) : c_v + (c - nq - nk)); };
  float sq = 0.f, sk = 0.f;
  constexpr int U = 4;  // channels a thread has in flight
  for (int c0 = threadIdx.x; c0 < C; c0 += U * blockDim.x) {
    float u[U][TMAX > 0 ? TMAX : 1], w[U][TMAX > 0 ? TMAX : 1], plain[U];
#pragma unroll
    for (int a = 0; a < U; ++a) {
      const int c = c0 + a * blockDim.x;
      const bool there = c < C;
      const int col = column(there ? c : 0);
      plain[a] = 0.f;
      if (TMAX == 0) {
        if (there) plain[a] = to_float(proj[(size_t)t * row + col]);
        continue;
      }
#pragma unroll
      for (int j = 0; j < TMAX; ++j) {
        const int back = taps - 1 - j, from = t - back;
        u[a][j] = w[a][j] = 0.f;
        if (there && j < taps && pos - back >= 0) {  // (before the sequence's first token: zeros)
          u[a][j] = from >= first ? to_float(proj[(size_t)from * row + col]) : srow[(size_t)(taps - 1 - (first - from)) * C + c];
          w[a][j] = conv_w[(size_t)c * taps + j];
        }
      }
    }
#pragma unroll
    for (int a = 0; a < U; ++a) {
      const int c = c0 + a * blockDim.x;
      if (c >= C) continue;
      float y = plain[a];
      if (TMAX > 0) {
        y = 0.f;
#pragma unroll
        for (int j = 0; j < TMAX; ++j) y = fmaf(w[a][j], u[a][j], y);  // (taps beyond the layer's, or before the sequence: zeros)
        y = to_float(from_float<T>(y));  // (the convolution's result in the activations' type, as a product's would be)
      }
      vals[c] = y;
      if (c < nq) sq = fmaf(y, y, sq);
      else if (c < nq + nk) sk = fmaf(y, y, sk);
    }
  }
  const float rq = rsqrtf(block_sum(sq, red) / (float)nq + eps);
  const float rk = rsqrtf(block_sum(sk, red) / (float)nk + eps);
  for (int c = threadIdx.x; c < nq + nk; c += blockDim.x) vals[c] *= c < nq ? rq * q_w[c] : rk * k_w[c - nq];
  __syncthreads();
  const int half = rotary / 2;
  const float* cs = rotary > 0 ? rope + (size_t)pos * rotary : nullptr;  // [2, half]
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float y = vals[c];
    if (c < nq + nk) {
      const int e = (c < nq ? c : c - nq) % d;
      if (e < rotary) {  // (u, v) -> (u cos - v sin, v cos + u sin) for the pair (i, i + half)
        const int i = e < half ? e : e - half;
        const float co = cs[i], si = cs[half + i];
        y = e < half ? vals[c] * co - vals[c + half] * si : vals[c] * co + vals[c - half] * si;
      }
    }
    if (c < nq) {
      q_out[(size_t)t * nq + c] = from_float<T>(y);
    } else if (c < nq + nk) {
      const int i = c - nq, kvh = i / d, e = i % d;
      k_cache[(((size_t)page * nkv + kvh) * bs + slot) * d + e] = from_float<T>(y);
    } else {
      const int i = c - nq - nk, kvh = i / dv, e = i % dv;
      v_cache[(((size_t)page * nkv + kvh) * dv + e) * bs + slot] = from_float<T>(y);
    }
  }
}

// Grid (items), a thread a channel in turns: row j of the new state is the projection at the position (end - (taps - 1) + j),
// from the step's tokens where the item brought it, else from the old row (shifted; read whole before it is written).
#define CS_MAX_TAPS 16
template <typename T>
__global__ __launch_bounds__(256) void conv_state_keep_kernel(const T* __restrict__ proj, long long row, int c_q, int c_k, int c_v,
                                                              float* __restrict__ state, const int* __restrict__ state_slots,
                                                              const int* __restrict__ item_start, int taps, int nq, int nk, int nv) {
  const int item = blockIdx.x, C = nq + nk + nv, keep = taps - 1;
  const int first = item_start[item], n = item_start[item + 1] - first;
  if (n <= 0) return;
  float* srow = state + (size_t)state_slots[item] * keep * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const int col = c < nq ? c_q + c : (c < nq + nk ? c_k + (c - nq) : c_v + (c - nq - nk));
    float next[CS_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CS_MAX_TAPS; ++j) {
      if (j >= keep) break;
      const int from = n - keep + j;  // the token of the item that row j holds afterwards (negative: a row of the old state)
      next[j] = from >= 0 ? to_float(proj[(size_t)(first + from) * row + col]) : srow[(size_t)(keep + from) * C + c];
    }
#pragma unroll
    for (int j = 0; j < CS_MAX_TAPS; ++j) {
      if (j >= keep) break;
      srow[(size_t)j * C + c] = next[j];
    }
  }
}

// proj [T, row] in the activations' type, q at column c_q (nh * d), k at c_k (nkv * d), v at c_v (nkv * dv). conv_w and state may be
// null with taps == 0; rope may be null with rotary == 0. q_out [T, nh * d].
extern "C" int me_conv_norm_rope_scatter(const void* proj, long long row, int c_q, int c_k, int c_v, const float* conv_w, int taps,
                                         float* state, const int* state_slots, const int* item_start, const float* q_w, const float* k_w,
                                         const float* rope, int rotary, const int* positions, const int* token_item,
                                         const int* block_table, int table_width, void* q_out, void* k_cache, void* v_cache,
                                         int num_tokens, int items, int nh, int nkv, int d, int dv, int bs, float eps, int dtype,
                                         hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (nh <= 0 || nkv <= 0 || d <= 0 || dv <= 0 || bs <= 0 || table_width <= 0)
    return me_fail("me_conv_norm_rope_scatter: heads %d / %d of %d and %d elements, pages of %d", nh, nkv, d, dv, bs);
  const long long nq = (long long)nh * d, nk = (long long)nkv * d, nv = (long long)nkv * dv, C = nq + nk + nv;
  if (c_q < 0 || c_k < 0 || c_v < 0 || c_q + nq > row || c_k + nk > row || c_v + nv > row)
    return me_fail("me_conv_norm_rope_scatter: columns %d, %d, %d of a row of %lld", c_q, c_k, c_v, row);
  if (taps < 0 || taps > CS_MAX_TAPS || (taps > 0 && !conv_w) || (taps > 1 && (!state || !state_slots)))
    return me_fail("me_conv_norm_rope_scatter: %d taps (0 to %d, with weights and, from 2 on, state rows)", taps, CS_MAX_TAPS);
  if (rotary < 0 || rotary % 2 || rotary > d || (rotary > 0 && !rope))
    return me_fail("me_conv_norm_rope_scatter: %d turned elements of a head of %d", rotary, d);
  const size_t lds = (size_t)C * sizeof(float);
  if (lds > 60 * 1024) return me_fail("me_conv_norm_rope_scatter: rows of %lld elements do not fit a block's memory", C);
  if (!item_start) return me_fail("me_conv_norm_rope_scatter: no item boundaries");
  // few tokens (decode steps): a block of 1,024 threads, so that a token's channels are fetched in one or two rounds
  const int threads = num_tokens <= 256 && C > 1024 ? 1024 : 256;
#define ME_CS_LAUNCH(TT, TM)                                                                                                          \
  conv_norm_rope_scatter_kernel<TT, TM><<<num_tokens, threads, lds, stream>>>(                                                          \
      (const TT*)proj, row, c_q, c_k, c_v, conv_w, taps, state, state_slots, item_start, q_w, k_w, rope, rotary, positions, token_item, \
      block_table, table_width, (TT*)q_out, (TT*)k_cache, (TT*)v_cache, nh, nkv, d, dv, bs, eps)
#define ME_CS_RUN(TT)                 \
  do {                                \
    if (taps == 0)                    \
      ME_CS_LAUNCH(TT, 0);            \
    else if (taps <= 4)               \
      ME_CS_LAUNCH(TT, 4);            \
    else if (taps <= 8)               \
      ME_CS_LAUNCH(TT, 8);            \
    else                              \
      ME_CS_LAUNCH(TT, CS_MAX_TAPS);  \
  } while (0)
  if (dtype == ME_F32) {
    ME_CS_RUN(float);
    if (taps > 1)
      conv_state_keep_kernel<float><<<items, 256, 0, stream>>>((const float*)proj, row, c_q, c_k, c_v, state, state_slots, item_start, taps,
                                                               (int)nq, (int)nk, (int)nv);
  } else {
    ME_CS_RUN(bf16_t);
    if (taps > 1)
      conv_state_keep_kernel<bf16_t><<<items, 256, 0, stream>>>((const bf16_t*)proj, row, c_q, c_k, c_v, state, state_slots, item_start,
                                                                taps, (int)nq, (int)nk, (int)nv);
  }
#undef ME_CS_RUN
#undef ME_CS_LAUNCH
  return me_check_launch("me_conv_norm_rope_scatter");
}
