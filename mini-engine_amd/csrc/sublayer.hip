// Row-wise kernels of a block that norms a sublayer's RESULT (not its input), x <- x + norm(sublayer(x)) * w, and of an input
// that every layer takes from the token itself.
//
//   result_norm_add  y = the sublayer's result of a token (a tensor in the activations' type, or float32 partial sums that are
//                    added up here in their order); x += scale * y * rsqrt(mean(y^2) + eps) * w; the new x is also written in
//                    the activations' type, which is what the next sublayer reads. With no result (the first sublayer of a
//                    model) it only writes x in the activations' type. Everything is float32 but that last rounding.
//   token_gate       out[t, j] = act(z[t, j]) * table[token_t, col0 + j]: a projection of the stream, through an activation,
//                    times a slice of a row that a table holds for every token id.
//   act_rows         out = act(in), elementwise: the activation of a feed-forward without a gate.
#include "common.h"

#define RN_HELD 8
template <typename T>
__global__ __launch_bounds__(256) void result_norm_add_kernel(float* __restrict__ x, const T* __restrict__ delta,
                                                              const float* __restrict__ parts, int num_parts, size_t part_stride,
                                                              const float* __restrict__ w, T* __restrict__ h, int dim, float eps,
                                                              float scale) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * dim;
  T* hr = h ? h + (size_t)t * dim : nullptr;
  if (!delta && !parts) {
    if (hr)
      for (int i = threadIdx.x; i < dim; i += blockDim.x) hr[i] = from_float<T>(xr[i]);
    return;
  }
  const T* dr = delta ? delta + (size_t)t * dim : nullptr;
  const float* pr = parts ? parts + (size_t)t * dim : nullptr;
  auto result_at = [&](int i) {
    if (dr) return to_float(dr[i]);
    float s = pr[i];
    for (int p = 1; p < num_parts; ++p) s += pr[(size_t)p * part_stride + i];
    return s;
  };
  float held[RN_HELD];  // the first RN_HELD * 256 elements of the row stay in registers between the two passes
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < RN_HELD; ++n) {
    const int i = threadIdx.x + 256 * n;
    held[n] = i < dim ? result_at(i) : 0.f;
    ss = fmaf(held[n], held[n], ss);
  }
  for (int i = threadIdx.x + 256 * RN_HELD; i < dim; i += 256) {
    const float y = result_at(i);
    ss = fmaf(y, y, ss);
  }
  const float r = rsqrtf(block_sum(ss, scratch) / (float)dim + eps) * scale;
#pragma unroll
  for (int n = 0; n < RN_HELD; ++n) {
    const int i = threadIdx.x + 256 * n;
    if (i < dim) {
      const float s = xr[i] + held[n] * r * w[i];
      xr[i] = s;
      if (hr) hr[i] = from_float<T>(s);
    }
  }
  for (int i = threadIdx.x + 256 * RN_HELD; i < dim; i += 256) {
    const float s = xr[i] + result_at(i) * r * w[i];
    xr[i] = s;
    if (hr) hr[i] = from_float<T>(s);
  }
}

// x float32 [T, dim] (updated in place); delta [T, dim] in the activations' type or null; parts float32 [num_parts, T, dim] or null
// (part_stride elements apart); w float32 [dim]; h [T, dim] in the activations' type or null.
extern "C" int me_result_norm_add(float* x, const void* delta, const float* parts, int num_parts, long long part_stride, const float* w,
                                  void* h, int num_tokens, int dim, float eps, float scale, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (dim <= 0) return me_fail("me_result_norm_add: dim=%d", dim);
  if ((delta || parts) && !w) return me_fail("me_result_norm_add: a result without a norm weight");
  if (parts && num_parts < 1) return me_fail("me_result_norm_add: %d partial sums", num_parts);
  if (dtype == ME_F32)
    result_norm_add_kernel<float><<<num_tokens, 256, 0, stream>>>(x, (const float*)delta, parts, num_parts, (size_t)part_stride, w,
                                                                   (float*)h, dim, eps, scale);
  else
    result_norm_add_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(x, (const bf16_t*)delta, parts, num_parts, (size_t)part_stride, w,
                                                                    (bf16_t*)h, dim, eps, scale);
  return me_check_launch("me_result_norm_add");
}

template <typename T>
__global__ __launch_bounds__(256) void token_gate_kernel(const T* __restrict__ z, const T* __restrict__ table, const int* __restrict__ ids,
                                                         const int* __restrict__ fed_rows, const int* __restrict__ fed_tokens,
                                                         T* __restrict__ out, int n, long long table_row, int col0, int vocab, int act,
                                                         long long total) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int t = (int)(i / n), j = (int)(i % n);
  int id = fed_rows && fed_rows[t] >= 0 ? fed_tokens[fed_rows[t]] : ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // ids are validated on the host; never fault
  const float e = to_float(table[(size_t)id * table_row + col0 + j]);
  out[i] = from_float<T>(ungated_act(to_float(z[i]), act) * e);
}

// z, out [T, n]; table [vocab, table_row] (all in the activations' type); ids int32 [T]; fed_rows / fed_tokens: where fed_rows[t] >= 0
// the id of token t is fed_tokens[fed_rows[t]] (both null: ids as they are). act: a code of MeAct.
extern "C" int me_token_gate(const void* z, const void* table, const int* ids, const int* fed_rows, const int* fed_tokens, void* out,
                             int num_tokens, int n, long long table_row, int col0, int vocab, int act, int dtype, hipStream_t stream) {
  if (num_tokens <= 0 || n <= 0) return 0;
  if (col0 < 0 || col0 + n > table_row || vocab <= 0) return me_fail("me_token_gate: columns %d .. %d of a row of %lld", col0, col0 + n - 1, table_row);
  if (!act_is_ungated(act)) return me_fail("me_token_gate: activation %d", act);
  const long long total = (long long)num_tokens * n;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == ME_F32)
    token_gate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)z, (const float*)table, ids, fed_rows, fed_tokens, (float*)out, n,
                                                         table_row, col0, vocab, act, total);
  else
    token_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)z, (const bf16_t*)table, ids, fed_rows, fed_tokens, (bf16_t*)out,
                                                          n, table_row, col0, vocab, act, total);
  return me_check_launch("me_token_gate");
}

template <typename T>
__global__ __launch_bounds__(256) void act_rows_kernel(const T* __restrict__ in, T* __restrict__ out, long long total, int act) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) out[i] = from_float<T>(ungated_act(to_float(in[i]), act));
}

extern "C" int me_act_rows(const void* in, void* out, long long total, int act, int dtype, hipStream_t stream) {
  if (total <= 0) return 0;
  if (!act_is_ungated(act)) return me_fail("me_act_rows: activation %d", act);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == ME_F32)
    act_rows_kernel<float><<<blocks, 256, 0, stream>>>((const float*)in, (float*)out, total, act);
  else
    act_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, total, act);
  return me_check_launch("me_act_rows");
}
