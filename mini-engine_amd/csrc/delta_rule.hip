// Linear attention by the generalized delta rule, with a matrix of state per request and head (float32):
//
//   u_t = k_t / sqrt(sum(k_t^2) + 1e-6)                                   the unit key
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T     both terms read the old state
//   o_t = S_t^T r_t
//
// with a decay per head and key channel w_t = exp(-c sigmoid(W_2 tanh(W_1 h_t) + w_0)) and a removal rate a_t =
// sigmoid(W_a h_t + b_a). Each head's o_t is divided by its root mean square, multiplied by a weight (all heads' size),
// by the sigmoid of a gate projection and by `out_scale`, and rounded to the activations' type.
//
// The projections of a token lie in one row of `proj` (r, k, v, gate, a: heads * d columns each; the inner product of
// the decay: `lora` columns), each at a column of its own. Everything behind the projections is float32: sigmoids,
// exponentials, the unit key, the state, the outputs and their norm.
//
// A block serves one (item, head) and walks the item's tokens in order. The state's column v (the value channel) belongs
// to four neighbouring lanes that hold its rows part, part + 4, ..: sums over the rows are a lane's own sum in ascending
// row, then two exchanges between neighbours, so their order depends on the head's size alone and a token's result has
// the same bits however the sequence was cut into steps and whatever else the step holds.
#include "common.h"

#define DR_PARTS 4
#define DR_MAX_D 256
#define DR_MAX_LORA 1024

__device__ __forceinline__ float dr_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }

template <typename T, int RPT>
__global__ __launch_bounds__(RPT * DR_PARTS * 4) void delta_rule_kernel(
    const T* __restrict__ proj, long long row, int c_r, int c_k, int c_v, int c_g, int c_a, int c_w1, const T* __restrict__ W2,
    const float* __restrict__ w0, const float* __restrict__ a_bias, const float* __restrict__ norm_w, float* __restrict__ state,
    const int* __restrict__ item_start, const int* __restrict__ state_slots, T* __restrict__ out, long long out_row, int out_col,
    float out_scale, int heads, int d, int lora, float eps, float decay_coef) {
  __shared__ float sk[DR_MAX_D], sv[DR_MAX_D], sr[DR_MAX_D], sw[DR_MAX_D], sa[DR_MAX_D], st[DR_MAX_LORA], red[16];
  const int item = blockIdx.x, head = blockIdx.y;
  const int slot = state_slots[item];
  if (slot < 0) return;
  const int tid = threadIdx.x, v = tid / DR_PARTS, part = tid % DR_PARTS;
  const bool column = v < d;
  float S[RPT];
  float* srow = state + ((size_t)slot * heads + head) * d * d;
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const int k = part + DR_PARTS * j;
    S[j] = column && k < d ? srow[(size_t)k * d + v] : 0.f;
  }
  const int hc = head * d;
  const int first = item_start[item], last = item_start[item + 1];
  for (int t = first; t < last; ++t) {
    const T* p = proj + (size_t)t * row;
    for (int j = tid; j < lora; j += blockDim.x) st[j] = tanhf(to_float(p[c_w1 + j]));
    __syncthreads();
    if (tid < d) {
      const int c = hc + tid;
      sk[tid] = to_float(p[c_k + c]);
      sv[tid] = to_float(p[c_v + c]);
      sr[tid] = to_float(p[c_r + c]);
      sa[tid] = dr_sigmoid(to_float(p[c_a + c]) + a_bias[c]);
      float z = w0[c];
      const T* w2 = W2 + (size_t)c * lora;
      for (int j = 0; j < lora; ++j) z = fmaf(to_float(w2[j]), st[j], z);
      sw[tid] = expf(-decay_coef * dr_sigmoid(z));
    }
    __syncthreads();
    // a lane's rows of the key: the sum of squares over all rows is the four neighbours' sums added up
    float kk[RPT], ss = 0.f;
#pragma unroll
    for (int j = 0; j < RPT; ++j) {
      const int k = part + DR_PARTS * j;
      kk[j] = k < d ? sk[k] : 0.f;
      ss = fmaf(kk[j], kk[j], ss);
    }
    ss += __shfl_xor(ss, 1, ME_WAVE);
    ss += __shfl_xor(ss, 2, ME_WAVE);
    const float inv = 1.f / sqrtf(ss + 1e-6f);
    float dot = 0.f;  // u^T S_(t-1) of this column
#pragma unroll
    for (int j = 0; j < RPT; ++j) dot = fmaf(kk[j] * inv, S[j], dot);
    dot += __shfl_xor(dot, 1, ME_WAVE);
    dot += __shfl_xor(dot, 2, ME_WAVE);
    const float vv = column ? sv[v] : 0.f;
    float o = 0.f;
#pragma unroll
    for (int j = 0; j < RPT; ++j) {
      const int k = part + DR_PARTS * j;
      if (k < d) {
        const float u = kk[j] * inv;
        S[j] = fmaf(kk[j], vv, fmaf(sw[k], S[j], -(sa[k] * u) * dot));
        o = fmaf(S[j], sr[k], o);
      }
    }
    o += __shfl_xor(o, 1, ME_WAVE);
    o += __shfl_xor(o, 2, ME_WAVE);
    const float sq = block_sum(column && part == 0 ? o * o : 0.f, red);
    if (column && part == 0) {
      const float g = dr_sigmoid(to_float(p[c_g + hc + v]));
      const float y = o * rsqrtf(sq / (float)d + eps) * norm_w[hc + v] * g * out_scale;
      out[(size_t)t * out_row + out_col + hc + v] = from_float<T>(y);
    }
    __syncthreads();  // the token's rows in LDS are read; the next token's may be written
  }
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const int k = part + DR_PARTS * j;
    if (column && k < d) srow[(size_t)k * d + v] = S[j];
  }
}

// proj [T, row]: the columns c_r, c_k, c_v, c_g, c_a (heads * d wide each) and c_w1 (`lora` wide). W2 [heads * d, lora] in the
// activations' type; w0, a_bias, norm_w float32 [heads * d]. state float32 [slots, heads, d, d]; item_start [items + 1],
// state_slots [items] (a negative slot: the item is skipped). out [T, out_row], written at the columns out_col ..
// out_col + heads * d - 1.
extern "C" int me_delta_rule(const void* proj, long long row, int c_r, int c_k, int c_v, int c_g, int c_a, int c_w1, const void* W2,
                             const float* w0, const float* a_bias, const float* norm_w, float* state, const int* item_start,
                             const int* state_slots, void* out, long long out_row, int out_col, float out_scale, int num_tokens,
                             int items, int heads, int d, int lora, float eps, float decay_coef, int dtype, hipStream_t stream) {
  if (num_tokens <= 0 || items <= 0) return 0;
  if (heads <= 0 || heads > 65535 || items > 65535 || d <= 0 || d > DR_MAX_D || lora <= 0 || lora > DR_MAX_LORA)
    return me_fail("me_delta_rule: heads=%d d=%d lora=%d items=%d (heads of up to %d elements, an inner size of up to %d)", heads, d,
                   lora, items, DR_MAX_D, DR_MAX_LORA);
  const long long hd = (long long)heads * d;
  const int cols[5] = {c_r, c_k, c_v, c_g, c_a};
  for (int c : cols)
    if (c < 0 || c + hd > row) return me_fail("me_delta_rule: a projection at column %d of a row of %lld", c, row);
  if (c_w1 < 0 || c_w1 + lora > row) return me_fail("me_delta_rule: the decay's inner projection at column %d of a row of %lld", c_w1, row);
  if (out_col < 0 || out_col + hd > out_row) return me_fail("me_delta_rule: the result at column %d of a row of %lld", out_col, out_row);
  const dim3 grid(items, heads);
#define DR_LAUNCH(TT, RPT)                                                                                                       \
  delta_rule_kernel<TT, RPT><<<grid, RPT * DR_PARTS * DR_PARTS, 0, stream>>>(                                                    \
      (const TT*)proj, row, c_r, c_k, c_v, c_g, c_a, c_w1, (const TT*)W2, w0, a_bias, norm_w, state, item_start, state_slots,     \
      (TT*)out, out_row, out_col, out_scale, heads, d, lora, eps, decay_coef)
#define DR_RUN(TT)            \
  do {                        \
    if (d <= 64)              \
      DR_LAUNCH(TT, 16);      \
    else if (d <= 128)        \
      DR_LAUNCH(TT, 32);      \
    else                      \
      DR_LAUNCH(TT, 64);      \
  } while (0)
  if (dtype == ME_F32)
    DR_RUN(float);
  else
    DR_RUN(bf16_t);
#undef DR_RUN
#undef DR_LAUNCH
  return me_check_launch("me_delta_rule");
}
