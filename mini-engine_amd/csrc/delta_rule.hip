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

#include <algorithm>

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
#pragma unroll 8
      for (int j = 0; j < lora; ++j) z = fmaf(to_float(w2[j]), st[j], z);  // (unrolled: eight loads on their way together)
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

// ---- steps that bring an item more than one token: four kernels, so that the walk over the tokens, which no token can start
// before the one ahead of it is done, does nothing but the recurrence.
//
//   prepare   every token at once: the decay w_t and the removal rate a_t (the inner product with W_2, sigmoids, the
//             exponential), and r_t, k_t, v_t as float32, laid out as the walk's lanes read them.
//   unit      every (token, head) at once: the unit key u_t and a_t * u_t.
//   scan      a wave of its own for every 4 value channels of an (item, head): the columns of the state do not meet, so the
//             waves of a head do not wait for each other, and a head of 64 channels keeps 16 compute units busy. A column
//             belongs to a row of 16 lanes that hold its rows part, part + 16, ..: sums over the rows are a lane's own sum,
//             then four exchanges inside the row of lanes (data-parallel moves, no trip through LDS), which leave every lane
//             of the row with the same bits. The vectors of the tokens ahead are asked for while this token's are multiplied
//             (SCAN_AHEAD tokens; what a lane holds of a token is a few registers).
//   finish    every token at once: a head's outputs over their root mean square, the weight, the gate, the scale.
//
// The sums over a column's rows run in another order than in the kernel above: a token's result differs from its by roundings.
// Within these kernels it does not depend on how the sequence was cut or on what else the step holds.
//
// Workspace, float32: [T, heads, 6, DP] with DP = 16 RPT >= d (k, u, w, a u, r in the lanes' order: row k at
// (k % 16) RPT + k / 16; then v in its own order; rows from d on are nought and leave the state's padding nought), then the
// raw outputs [T, heads, d rounded up to a multiple of 4].
#define DS_PARTS 16
#define DS_VECS 6

template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(const T* __restrict__ proj, long long row, int c_r, int c_k, int c_v, int c_a,
                                                            int c_w1, const T* __restrict__ W2, const float* __restrict__ w0,
                                                            const float* __restrict__ a_bias, float* __restrict__ ws, int num_tokens,
                                                            int heads, int d, int lora, int rpt, float decay_coef) {
  constexpr int TT = 8;  // tokens a block: a thread reads its row of W_2 once for all of them
  __shared__ float st[TT][DR_MAX_LORA];
  const int t0 = blockIdx.x * TT, tokens = min(TT, num_tokens - t0);
  const int hd = heads * d, dp = rpt * DS_PARTS;
  for (int i = threadIdx.x; i < TT * lora; i += blockDim.x) {
    const int tt = i / lora, j = i % lora;
    st[tt][j] = tt < tokens ? tanhf(to_float(proj[(size_t)(t0 + tt) * row + c_w1 + j])) : 0.f;
  }
  __syncthreads();
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < hd; c += gridDim.y * blockDim.x) {
    const int head = c / d, k = c % d;
    const int place = (k % DS_PARTS) * rpt + k / DS_PARTS;  // where the lane that owns row k finds it
    float z[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) z[tt] = w0[c];
    const T* w2 = W2 + (size_t)c * lora;
    for (int j = 0; j < lora; ++j) {
      const float wj = to_float(w2[j]);
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) z[tt] = fmaf(wj, st[tt][j], z[tt]);
    }
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      if (tt < tokens) {
        const T* p = proj + (size_t)(t0 + tt) * row;
        float* o = ws + ((size_t)(t0 + tt) * heads + head) * DS_VECS * dp;
        o[place] = to_float(p[c_k + c]);
        o[2 * dp + place] = expf(-decay_coef * dr_sigmoid(z[tt]));
        o[3 * dp + place] = dr_sigmoid(to_float(p[c_a + c]) + a_bias[c]);
        o[4 * dp + place] = to_float(p[c_r + c]);
        o[5 * dp + k] = to_float(p[c_v + c]);
      }
    }
  }
}

// Rows from d on of the workspace's vectors: nought (once a step, before the other kernels fill the rest).
__global__ __launch_bounds__(256) void delta_pad_kernel(float* __restrict__ ws, long long units, int d, int rpt) {
  const int dp = rpt * DS_PARTS, pad = dp - d;
  const long long n = units * DS_VECS * pad;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    const long long vec = i / pad;
    const int k = d + (int)(i % pad);
    const int place = vec % DS_VECS == 5 ? k : (k % DS_PARTS) * rpt + k / DS_PARTS;
    ws[vec * dp + place] = 0.f;
  }
}

// Grid (tokens, heads), a wave each: u = k / sqrt(sum(k^2) + 1e-6) and a u (in a's place).
__global__ __launch_bounds__(64) void delta_unit_kernel(float* __restrict__ ws, int heads, int rpt) {
  const int dp = rpt * DS_PARTS;
  float* p = ws + ((size_t)blockIdx.x * heads + blockIdx.y) * DS_VECS * dp;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dp; i += 64) ss = fmaf(p[i], p[i], ss);  // (the padding adds nought)
  const float inv = 1.f / sqrtf(wave_sum(ss) + 1e-6f);
  for (int i = threadIdx.x; i < dp; i += 64) {
    const float u = p[i] * inv;
    p[dp + i] = u;
    p[3 * dp + i] *= u;
  }
}

template <int RPT>
struct DeltaRows {
  float k[RPT], u[RPT], w[RPT], au[RPT], r[RPT], v;
};

template <int RPT>
__device__ __forceinline__ void delta_fetch(DeltaRows<RPT>& x, const float* __restrict__ p, int part, int v) {
  constexpr int DP = RPT * DS_PARTS;
  float* dst[5] = {x.k, x.u, x.w, x.au, x.r};
#pragma unroll
  for (int vec = 0; vec < 5; ++vec) {
    const float4* src = reinterpret_cast<const float4*>(p + vec * DP + part * RPT);
#pragma unroll
    for (int q = 0; q < RPT / 4; ++q) {
      const float4 a = src[q];
      dst[vec][4 * q] = a.x, dst[vec][4 * q + 1] = a.y, dst[vec][4 * q + 2] = a.z, dst[vec][4 * q + 3] = a.w;
    }
  }
  x.v = p[5 * DP + v];
}

// The sum of a value over the 16 lanes of its row, in every lane of the row (the same bits in all of them: a rotation by 8,
// one by 4, then the two exchanges inside a group of four add the same pairs in every lane).
__device__ __forceinline__ float row16_sum(float x) {
#define DS_DPP_ADD(CTRL) x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false))
  DS_DPP_ADD(0x128);  // row_ror:8
  DS_DPP_ADD(0x124);  // row_ror:4
  DS_DPP_ADD(0x4e);   // quad_perm:[2,3,0,1]
  DS_DPP_ADD(0xb1);   // quad_perm:[1,0,3,2]
#undef DS_DPP_ADD
  return x;
}

// One token of the recurrence for a lane's rows of its column.
template <int RPT>
__device__ __forceinline__ float delta_token(float (&S)[RPT], const DeltaRows<RPT>& x) {
  // (two sums side by side, even rows and odd rows: a wave that walks the tokens alone waits for every result it needs next)
  float dot0 = 0.f, dot1 = 0.f;
#pragma unroll
  for (int j = 0; j < RPT; j += 2) {
    dot0 = fmaf(x.u[j], S[j], dot0);
    dot1 = fmaf(x.u[j + 1], S[j + 1], dot1);
  }
  const float dot = row16_sum(dot0 + dot1);
  float o0 = 0.f, o1 = 0.f;
#pragma unroll
  for (int j = 0; j < RPT; j += 2) {
    S[j] = fmaf(x.k[j], x.v, fmaf(x.w[j], S[j], -x.au[j] * dot));
    S[j + 1] = fmaf(x.k[j + 1], x.v, fmaf(x.w[j + 1], S[j + 1], -x.au[j + 1] * dot));
    o0 = fmaf(S[j], x.r[j], o0);
    o1 = fmaf(S[j + 1], x.r[j + 1], o1);
  }
  return row16_sum(o0 + o1);
}

template <int RPT, int AHEAD>
__global__ __launch_bounds__(64) void delta_scan_kernel(const float* __restrict__ ws, float* __restrict__ state,
                                                        const int* __restrict__ item_start, const int* __restrict__ state_slots,
                                                        float* __restrict__ raw, int heads, int d) {
  constexpr int DP = RPT * DS_PARTS;
  const int item = blockIdx.x, head = blockIdx.y;
  const int slot = state_slots[item];
  if (slot < 0) return;
  const int lane = threadIdx.x, v = blockIdx.z * 4 + lane / DS_PARTS, part = lane % DS_PARTS;
  const bool column = v < d;
  const int vv = column ? v : 0;  // (a lane beyond the head's columns reads a real one; what it stores lands in the padding of the raw outputs)
  float S[RPT];
  float* srow = state + ((size_t)slot * heads + head) * d * d;
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const int k = part + DS_PARTS * j;
    S[j] = column && k < d ? srow[(size_t)k * d + v] : 0.f;
  }
  const int first = item_start[item], last = item_start[item + 1];
  if (first >= last) return;
  const int dpad = 4 * ((d + 3) / 4);  // the raw outputs' rows hold whole groups of four columns: every lane stores, no lane branches
  const size_t step = (size_t)heads * DS_VECS * DP, hd = (size_t)heads * dpad;
  const float* p = ws + ((size_t)first * heads + head) * DS_VECS * DP;
  float* out = raw + (size_t)first * hd + (size_t)head * dpad + v;
  DeltaRows<RPT> x[AHEAD];
#pragma unroll
  for (int b = 0; b < AHEAD; ++b) delta_fetch<RPT>(x[b], p + (size_t)min(b, last - 1 - first) * step, part, vv);
  // AHEAD tokens a turn, without a branch between them (a token's output is summed and stored while the next token's sums
  // begin; the compiler moves instructions only inside a stretch without branches): a token's vectors are asked for AHEAD tokens
  // ahead, those beyond the item's last token at the last token's place (fetched and not used).
  int t = first;
  for (; t + AHEAD <= last; t += AHEAD) {
#pragma unroll
    for (int b = 0; b < AHEAD; ++b) {
      out[b * hd] = delta_token<RPT>(S, x[b]);  // (the 16 lanes of a column store the same number to the same place)
      delta_fetch<RPT>(x[b], p + (size_t)min(b + AHEAD, last - 1 - t) * step, part, vv);
    }
    p += AHEAD * step;
    out += AHEAD * hd;
  }
#pragma unroll
  for (int b = 0; b < AHEAD; ++b)
    if (t + b < last) out[b * hd] = delta_token<RPT>(S, x[b]);
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const int k = part + DS_PARTS * j;
    if (column && k < d) srow[(size_t)k * d + v] = S[j];
  }
}

// Grid (tokens, heads), a wave each.
template <typename T>
__global__ __launch_bounds__(64) void delta_finish_kernel(const float* __restrict__ raw, const T* __restrict__ proj, long long row, int c_g,
                                                          const float* __restrict__ norm_w, T* __restrict__ out, long long out_row,
                                                          int out_col, float out_scale, int heads, int d, float eps) {
  const int t = blockIdx.x, head = blockIdx.y, hc = head * d;
  const float* o = raw + ((size_t)t * heads + head) * (4 * ((d + 3) / 4));
  float sq = 0.f;
  for (int v = threadIdx.x; v < d; v += 64) sq = fmaf(o[v], o[v], sq);
  sq = wave_sum(sq);
  const float inv = rsqrtf(sq / (float)d + eps);
  const T* p = proj + (size_t)t * row + c_g + hc;
  T* y = out + (size_t)t * out_row + out_col + hc;
  for (int v = threadIdx.x; v < d; v += 64) y[v] = from_float<T>(o[v] * inv * norm_w[hc + v] * dr_sigmoid(to_float(p[v])) * out_scale);
}

static int delta_rows_per_lane(int d) { return 4 * ((d + 4 * DS_PARTS - 1) / (4 * DS_PARTS)); }  // 4, 8, 12 or 16

// Bytes of workspace that me_delta_rule_steps needs for a step of `tokens` tokens.
extern "C" long long me_delta_rule_workspace(long long tokens, int heads, int d) {
  if (tokens <= 0 || heads <= 0 || d <= 0 || d > DR_MAX_D) return 0;
  const long long dp = (long long)delta_rows_per_lane(d) * DS_PARTS;
  return (tokens * heads * DS_VECS * dp + tokens * heads * (4 * ((d + 3) / 4))) * 4 + 256;
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

// As me_delta_rule, by the three kernels for steps that bring an item more than one token; ws: me_delta_rule_workspace bytes.
extern "C" int me_delta_rule_steps(const void* proj, long long row, int c_r, int c_k, int c_v, int c_g, int c_a, int c_w1, const void* W2,
                                   const float* w0, const float* a_bias, const float* norm_w, float* state, const int* item_start,
                                   const int* state_slots, void* out, long long out_row, int out_col, float out_scale, int num_tokens,
                                   int items, int heads, int d, int lora, float eps, float decay_coef, int dtype, void* workspace,
                                   hipStream_t stream) {
  if (num_tokens <= 0 || items <= 0) return 0;
  if (heads <= 0 || heads > 65535 || items > 65535 || d <= 0 || d > DR_MAX_D || lora <= 0 || lora > DR_MAX_LORA)
    return me_fail("me_delta_rule_steps: heads=%d d=%d lora=%d items=%d (heads of up to %d elements, an inner size of up to %d)", heads,
                   d, lora, items, DR_MAX_D, DR_MAX_LORA);
  const long long hd = (long long)heads * d;
  const int cols[5] = {c_r, c_k, c_v, c_g, c_a};
  for (int c : cols)
    if (c < 0 || c + hd > row) return me_fail("me_delta_rule_steps: a projection at column %d of a row of %lld", c, row);
  if (c_w1 < 0 || c_w1 + lora > row)
    return me_fail("me_delta_rule_steps: the decay's inner projection at column %d of a row of %lld", c_w1, row);
  if (out_col < 0 || out_col + hd > out_row) return me_fail("me_delta_rule_steps: the result at column %d of a row of %lld", out_col, out_row);
  if (!workspace || ((uintptr_t)workspace & 15)) return me_fail("me_delta_rule_steps: a workspace at a multiple of 16 bytes");
  const int rpt = delta_rows_per_lane(d), dp = rpt * DS_PARTS;
  float* ws = (float*)workspace;
  float* raw = ws + (size_t)num_tokens * heads * DS_VECS * dp;
  if (dp > d) {
    const long long n = (long long)num_tokens * heads * DS_VECS * (dp - d);
    delta_pad_kernel<<<(unsigned)std::min<long long>((n + 255) / 256, 4096), 256, 0, stream>>>(ws, (long long)num_tokens * heads, d, rpt);
  }
  const dim3 pgrid((num_tokens + 7) / 8, (unsigned)std::min<long long>((hd + 255) / 256, 64));
  const dim3 sgrid(items, heads, (d + 3) / 4), tgrid(num_tokens, heads);
  if (dtype == ME_F32)
    delta_prepare_kernel<float><<<pgrid, 256, 0, stream>>>((const float*)proj, row, c_r, c_k, c_v, c_a, c_w1, (const float*)W2, w0, a_bias,
                                                           ws, num_tokens, heads, d, lora, rpt, decay_coef);
  else
    delta_prepare_kernel<bf16_t><<<pgrid, 256, 0, stream>>>((const bf16_t*)proj, row, c_r, c_k, c_v, c_a, c_w1, (const bf16_t*)W2, w0,
                                                            a_bias, ws, num_tokens, heads, d, lora, rpt, decay_coef);
  delta_unit_kernel<<<tgrid, 64, 0, stream>>>(ws, heads, rpt);
  switch (rpt) {
    case 4:  // (the further ahead a token's vectors are asked for, the less of their way from memory is waited for)
      delta_scan_kernel<4, 8><<<sgrid, 64, 0, stream>>>(ws, state, item_start, state_slots, raw, heads, d);
      break;
    case 8:
      delta_scan_kernel<8, 4><<<sgrid, 64, 0, stream>>>(ws, state, item_start, state_slots, raw, heads, d);
      break;
    case 12:
      delta_scan_kernel<12, 2><<<sgrid, 64, 0, stream>>>(ws, state, item_start, state_slots, raw, heads, d);
      break;
    default:
      delta_scan_kernel<16, 2><<<sgrid, 64, 0, stream>>>(ws, state, item_start, state_slots, raw, heads, d);
  }
  if (dtype == ME_F32)
    delta_finish_kernel<float><<<tgrid, 64, 0, stream>>>(raw, (const float*)proj, row, c_g, norm_w, (float*)out, out_row, out_col, out_scale,
                                                         heads, d, eps);
  else
    delta_finish_kernel<bf16_t><<<tgrid, 64, 0, stream>>>(raw, (const bf16_t*)proj, row, c_g, norm_w, (bf16_t*)out, out_row, out_col,
                                                          out_scale, heads, d, eps);
  return me_check_launch("me_delta_rule_steps");
}
