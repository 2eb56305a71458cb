// Attention over one latent per token (keys and values of all heads are linear maps of it), in the form that never
// expands the latents: with c the normed latent [rank] and k_r the rotated key part [r] that all heads share,
//   score_h(i, j) = q_h[:d] . (W_uk_h c_j) + rot(q_h[d:]) . k_r_j = (W_uk_h^T q_h[:d]) . c_j + rot(q_h[d:]) . k_r_j
//   out_h(i)      = W_uv_h (sum_j p_h(i, j) c_j)
// so a layer caches one key [c | k_r] per token (one key/value head for all query heads) whose first `rank` elements
// are also its value. The kernels here prepare that: the latent's norm, the rotation, the page write, and the two small
// products per head (W_uk_h^T on the queries, W_uv_h on the weighted latents, with the output gate). The attention
// itself is the framework's, over a page pool with one key/value head.
#include "tile_product.h"

// proj [T, row_stride]: nh query heads of (d + r), then rank + r elements of the latent projection (what follows in the
// row is not read here). One block per token:
//   c = latent[:rank] * rsqrt(mean(latent[:rank]^2) + eps) * norm_w  -> K[page, 0, slot, :rank], V[page, 0, :rank, slot]
//   k_r = latent[rank:] turned by the position's angles (element i with i + r/2)  -> K[page, 0, slot, rank:]
//   (with value rows for the whole key, v_rows == rank + r, also V[page, 0, rank:, slot])
//   every head's q[d:] turned likewise -> qa[t, h, rank:]   (qa [T, nh, rank + r]; its first rank elements are the
//   product of the kernel below)
// rope: float32 [positions, 2, r/2], cosines then sines, already multiplied by whatever the encoding multiplies them by.
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ proj, size_t row_stride, const float* __restrict__ norm_w, const float* __restrict__ rope,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table, int table_width,
    T* __restrict__ qa, T* __restrict__ k_cache, T* __restrict__ v_cache, int nh, int d, int r, int rank, int v_rows, int bs,
    float eps, int writes) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, dk = rank + r, half = r / 2;
  const int pos = positions[t];
  const int page = writes ? block_table[(size_t)token_item[t] * table_width + pos / bs] : -1, slot = pos % bs;
  const T* row = proj + (size_t)t * row_stride;
  const T* lat = row + (size_t)nh * (d + r);
  float ss = 0.f;
  if (writes)  // (a layer that reads another layer's pages has no latent projection: its rows hold the queries alone)
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
      const float v = to_float(lat[i]);
      ss = fmaf(v, v, ss);
    }
  const float inv = writes ? rsqrtf(block_sum(ss, scratch) / (float)rank + eps) : 0.f;
  const float* cs = rope + (size_t)pos * r;
  if (page >= 0) {
    T* krow = k_cache + ((size_t)page * bs + slot) * dk;
    T* vcol = v_cache + (size_t)page * v_rows * bs + slot;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
      const T c = from_float<T>(to_float(lat[i]) * inv * norm_w[i]);
      krow[i] = c;
      vcol[(size_t)i * bs] = c;
    }
    for (int i = threadIdx.x; i < r; i += blockDim.x) {
      const bool first = i < half;
      const int j = first ? i : i - half;
      const float a = to_float(lat[rank + i]), b = to_float(lat[rank + (first ? i + half : i - half)]);
      const T v = from_float<T>(first ? a * cs[j] - b * cs[half + j] : a * cs[j] + b * cs[half + j]);
      krow[rank + i] = v;
      if (v_rows == dk) vcol[(size_t)(rank + i) * bs] = v;
    }
  }
  for (int idx = threadIdx.x; idx < nh * r; idx += blockDim.x) {
    const int h = idx / r, i = idx % r;
    const T* src = row + (size_t)h * (d + r) + d;
    const bool first = i < half;
    const int j = first ? i : i - half;
    const float a = to_float(src[i]), b = to_float(src[first ? i + half : i - half]);
    qa[((size_t)t * nh + h) * dk + rank + i] = from_float<T>(first ? a * cs[j] - b * cs[half + j] : a * cs[j] + b * cs[half + j]);
  }
}

// writes == 0: the layer reads another layer's pages; its rows hold no latent projection (queries, then whatever follows), nothing
// is normed and no page is written, only the queries' turned parts.
extern "C" int me_latent_prepare_for(const void* proj, long long row_stride, const float* norm_w, const float* rope,
                                     const int* positions, const int* token_item, const int* block_table, int table_width, void* qa,
                                     void* k_cache, void* v_cache, int num_tokens, int nh, int d, int r, int rank, int v_rows, int bs,
                                     float eps, int writes, int dtype, hipStream_t stream);

extern "C" int me_latent_prepare(const void* proj, long long row_stride, const float* norm_w, const float* rope,
                                 const int* positions, const int* token_item, const int* block_table, int table_width, void* qa,
                                 void* k_cache, void* v_cache, int num_tokens, int nh, int d, int r, int rank, int v_rows, int bs,
                                 float eps, int dtype, hipStream_t stream) {
  return me_latent_prepare_for(proj, row_stride, norm_w, rope, positions, token_item, block_table, table_width, qa, k_cache, v_cache,
                               num_tokens, nh, d, r, rank, v_rows, bs, eps, 1, dtype, stream);
}

extern "C" int me_latent_prepare_for(const void* proj, long long row_stride, const float* norm_w, const float* rope,
                                     const int* positions, const int* token_item, const int* block_table, int table_width, void* qa,
                                     void* k_cache, void* v_cache, int num_tokens, int nh, int d, int r, int rank, int v_rows, int bs,
                                     float eps, int writes, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (nh <= 0 || d <= 0 || rank <= 0 || r <= 0 || r % 2) return me_fail("me_latent_prepare: heads=%d d=%d rank=%d rot=%d", nh, d, rank, r);
  if (v_rows != rank && v_rows != rank + r) return me_fail("me_latent_prepare: value pages of %d rows for a latent of %d + %d", v_rows, rank, r);
  if (row_stride < (long long)nh * (d + r) + (writes ? rank + r : 0)) return me_fail("me_latent_prepare: rows of %lld elements are too short", row_stride);
  if (bs <= 0 || table_width <= 0) return me_fail("me_latent_prepare: block_size=%d table_width=%d", bs, table_width);
  if (dtype == ME_F32)
    latent_prepare_kernel<float><<<num_tokens, 256, 0, stream>>>((const float*)proj, (size_t)row_stride, norm_w, rope, positions,
                                                                 token_item, block_table, table_width, (float*)qa, (float*)k_cache,
                                                                 (float*)v_cache, nh, d, r, rank, v_rows, bs, eps, writes);
  else
    latent_prepare_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((const bf16_t*)proj, (size_t)row_stride, norm_w, rope, positions,
                                                                  token_item, block_table, table_width, (bf16_t*)qa,
                                                                  (bf16_t*)k_cache, (bf16_t*)v_cache, nh, d, r, rank, v_rows, bs, eps, writes);
  return me_check_launch("me_latent_prepare");
}

// A product per head: out[t, h, j] = sum_i x[t, h, i] W[h, j, i] for j < n, i < k, times sigmoid(gate[t, h]) if a gate is
// given. x, out and gate are addressed by strides in elements (row = token, head), so they may be slices of wider rows.
// Grid (tiles of 16 tokens, tiles of 64 columns, heads).
template <typename T>
__global__ __launch_bounds__(256) void head_product_kernel(const T* __restrict__ x, size_t x_row, size_t x_head,
                                                           const T* __restrict__ W, T* __restrict__ out, size_t out_row,
                                                           size_t out_head, const T* __restrict__ gate, size_t gate_row,
                                                           int num_tokens, int n, int k) {
  __shared__ TileLds lds;
  const int t0 = blockIdx.x * TP_ROWS, c0 = blockIdx.y * TP_COLS, h = blockIdx.z;
  const int rows = min(TP_ROWS, num_tokens - t0), cols = min(TP_COLS, n - c0);
  float acc[4];
  tile_product<T>([&](int i) { return x + (size_t)(t0 + i) * x_row + (size_t)h * x_head; }, rows, W + ((size_t)h * n + c0) * k,
                  cols, k, acc, lds);
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  if (tx >= cols) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = ty + 4 * i;
    if (row < rows) {
      float v = acc[i];
      if (gate) v *= 1.f / (1.f + expf(-to_float(gate[(size_t)(t0 + row) * gate_row + h])));
      out[(size_t)(t0 + row) * out_row + (size_t)h * out_head + c0 + tx] = from_float<T>(v);
    }
  }
}

// The same on the matrix cores (bfloat16; k and all strides multiples of 8 elements, bases at multiples of 16 bytes): a block
// takes 16 * MT tokens and 64 columns of a head, a wave 16 columns (tile_product.h: wave_product_bf16).
template <int MT>
__global__ __launch_bounds__(256) void head_product_mfma_kernel(const bf16_t* __restrict__ x, size_t x_row, size_t x_head,
                                                                const bf16_t* __restrict__ W, bf16_t* __restrict__ out, size_t out_row,
                                                                size_t out_head, const bf16_t* __restrict__ gate, size_t gate_row,
                                                                int num_tokens, int n, int k) {
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1), r = lane & 15, g = lane >> 4;
  const int t0 = blockIdx.x * 16 * MT, n0 = blockIdx.y * 64 + wave * 16, h = blockIdx.z;
  if (n0 >= n) return;
  const bf16_t* wrow[1] = {n0 + r < n ? W + ((size_t)h * n + n0 + r) * k : nullptr};
  const bf16_t* xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int tok = t0 + t * 16 + r;
    xrow[t] = tok < num_tokens ? x + (size_t)tok * x_row + (size_t)h * x_head : nullptr;
  }
  tp_float4 acc[MT][1];
  wave_product_bf16<MT, 1>(xrow, wrow, k, acc);
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int tok = t0 + t * 16 + r;
    if (tok >= num_tokens) continue;
    const float gv = gate ? 1.f / (1.f + expf(-to_float(gate[(size_t)tok * gate_row + h]))) : 1.f;
    bf16_t* dst = out + (size_t)tok * out_row + (size_t)h * out_head + n0 + 4 * g;
    if (n0 + 4 * g + 3 < n && (((uintptr_t)dst) & 7) == 0) {  // the lane's four columns as one store
      typedef __bf16 hp_bf16x4 __attribute__((ext_vector_type(4)));
      const hp_bf16x4 v = {(__bf16)(acc[t][0][0] * gv), (__bf16)(acc[t][0][1] * gv), (__bf16)(acc[t][0][2] * gv), (__bf16)(acc[t][0][3] * gv)};
      *reinterpret_cast<hp_bf16x4*>(dst) = v;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n0 + 4 * g + i < n) dst[i] = from_float<bf16_t>(acc[t][0][i] * gv);
    }
  }
}

extern "C" int me_head_product(const void* x, long long x_row, long long x_head, const void* W, void* out, long long out_row,
                               long long out_head, const void* gate, long long gate_row, int num_tokens, int heads, int n, int k,
                               int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (heads <= 0 || heads > 65535 || n <= 0 || k <= 0) return me_fail("me_head_product: heads=%d n=%d k=%d", heads, n, k);
  const dim3 grid((num_tokens + TP_ROWS - 1) / TP_ROWS, (n + TP_COLS - 1) / TP_COLS, heads);
  if (grid.y > 65535) return me_fail("me_head_product: %d columns a head", n);
  if (dtype == ME_BF16 && k % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0 && (((uintptr_t)x | (uintptr_t)W) & 15) == 0) {
    if (num_tokens >= 64)
      head_product_mfma_kernel<4><<<dim3((num_tokens + 63) / 64, grid.y, heads), 256, 0, stream>>>(
          (const bf16_t*)x, (size_t)x_row, (size_t)x_head, (const bf16_t*)W, (bf16_t*)out, (size_t)out_row, (size_t)out_head,
          (const bf16_t*)gate, (size_t)gate_row, num_tokens, n, k);
    else
      head_product_mfma_kernel<1><<<grid, 256, 0, stream>>>((const bf16_t*)x, (size_t)x_row, (size_t)x_head, (const bf16_t*)W,
                                                            (bf16_t*)out, (size_t)out_row, (size_t)out_head, (const bf16_t*)gate,
                                                            (size_t)gate_row, num_tokens, n, k);
    return me_check_launch("me_head_product");
  }
  if (dtype == ME_F32)
    head_product_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, (size_t)x_row, (size_t)x_head, (const float*)W, (float*)out,
                                                         (size_t)out_row, (size_t)out_head, (const float*)gate, (size_t)gate_row,
                                                         num_tokens, n, k);
  else
    head_product_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, (size_t)x_row, (size_t)x_head, (const bf16_t*)W,
                                                          (bf16_t*)out, (size_t)out_row, (size_t)out_head, (const bf16_t*)gate,
                                                          (size_t)gate_row, num_tokens, n, k);
  return me_check_launch("me_head_product");
}

// rows [T, heads, n] in place: head h of token t times sigmoid(gate[t, h]) (gate addressed by its row stride).
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ rows, const T* __restrict__ gate, size_t gate_row, int heads, int n, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t unit = i / n;
  const size_t t = unit / heads, h = unit % heads;
  const float g = 1.f / (1.f + expf(-to_float(gate[t * gate_row + h])));
  rows[i] = from_float<T>(to_float(rows[i]) * g);
}

extern "C" int me_head_gate(void* rows, const void* gate, long long gate_row, int num_tokens, int heads, int n, int dtype,
                            hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (heads <= 0 || n <= 0) return me_fail("me_head_gate: heads=%d n=%d", heads, n);
  const size_t total = (size_t)num_tokens * heads * n;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == ME_F32)
    head_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)rows, (const float*)gate, (size_t)gate_row, heads, n, total);
  else
    head_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)rows, (const bf16_t*)gate, (size_t)gate_row, heads, n, total);
  return me_check_launch("me_head_gate");
}

// A decode step's tail of a latent attention layer in one kernel: the sum over the splits of the split-context attention
// kernel (their unnormalised weighted latents part_o [item, head, split, dk] and statistics part_ml [.., 2] = (maximum in
// units of log2, sum), with the sink as one more split of weight 1 and no value), the result rounded to bfloat16 as the
// kernel that adds up splits rounds it, then the head's values' map and its gate:
//   out[item, head, :] = sigmoid(gate[item, head]) * W_uv[head] . round(sum_s w_s o_s[:rank] / sum_s w_s l_s)
// One block of 256 threads per (item, head).
#define LV_MAX_SPLITS 1024
#define LV_MAX_RANK 512
__global__ __launch_bounds__(256) void latent_values_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                            int num_splits, int dk, int rank, const float* __restrict__ sink,
                                                            const bf16_t* __restrict__ W_uv, const bf16_t* __restrict__ gate,
                                                            size_t gate_row, bf16_t* __restrict__ out, int nh, int dv) {
  __shared__ float wgt[LV_MAX_SPLITS];
  __shared__ __attribute__((aligned(16))) float lat[LV_MAX_RANK];
  __shared__ __attribute__((aligned(16))) bf16_t latb[LV_MAX_RANK];  // the same, as the matrix cores read it
  __shared__ float4 partial[256];
  __shared__ float red_max[4], red_sum[4];
  const size_t unit = blockIdx.x;
  const int item = (int)(unit / nh), head = (int)(unit % nh);
  const int tid = threadIdx.x, lane = tid & (ME_WAVE - 1), wave = tid / ME_WAVE;
  const float* ml = part_ml + unit * num_splits * 2;
  const float* po = part_o + unit * num_splits * dk;
  // what nothing has to be waited for is asked for first: this thread's first weights of the values' map, and its first
  // partial results (thread -> four elements of the latent, one of 256 / (rank / 4) groups of splits)
  constexpr int EARLY = 8;
  // Loads come back in the order they were asked for: first what the kernel needs first (this thread's split's statistics and
  // the sink), then its partial results, then the weights and the gate, which wait for the kernel's end.
  const float m_mine = tid < num_splits ? ml[tid * 2] : -INFINITY, l_mine = tid < num_splits ? ml[tid * 2 + 1] : 0.f;
  const float sink_raw = sink ? sink[head] : 0.f;
  const bool wide = rank % 8 == 0 && (((uintptr_t)W_uv) & 15) == 0;
  // (the values' map on the matrix cores: wave w takes the tiles of 16 columns w, w + 4, ..; lane (r, g) feeds row n0 + r of the
  // map, eight elements from 32 c + 8 g; the one token's latent is row 0 of the other operand)
  const int rr = lane & 15, gg = lane >> 4;
  const bf16_t* wrow = wave * 16 + rr < dv ? W_uv + ((size_t)head * dv + wave * 16 + rr) * rank : nullptr;
  const bool quads_ok = rank % 4 == 0 && dk % 4 == 0 && rank / 4 <= 256;
  const int quads = quads_ok ? rank / 4 : 1, groups = quads_ok ? 256 / quads : 1;
  const int qd = tid % quads, grp = tid / quads;
  float4 early[EARLY];
#pragma unroll
  for (int i = 0; i < EARLY; ++i) {
    const int sp = grp + i * groups;
    early[i] = quads_ok && grp < groups && sp < num_splits ? *reinterpret_cast<const float4*>(po + (size_t)sp * dk + qd * 4)
                                                           : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  tp_bf16x8 wpre[EARLY];
#pragma unroll
  for (int i = 0; i < EARLY; ++i) {
    wpre[i] = tp_bf16x8{};
    if (wide && wrow && 32 * i + 8 * gg < rank) wpre[i] = *reinterpret_cast<const tp_bf16x8*>(wrow + 32 * i + 8 * gg);
  }
  const float gate_raw = gate ? to_float(gate[(size_t)item * gate_row + head]) : 0.f;
  float big = l_mine > 0.f ? m_mine : -INFINITY;
  for (int s = tid + 256; s < num_splits; s += 256)
    if (ml[s * 2 + 1] > 0.f) big = fmaxf(big, ml[s * 2]);
  big = wave_max(big);
  if (lane == 0) red_max[wave] = big;
  __syncthreads();
  big = fmaxf(fmaxf(red_max[0], red_max[1]), fmaxf(red_max[2], red_max[3]));
  const float s2 = sink ? sink_raw * 1.4426950408889634f : -INFINITY;
  big = fmaxf(big, s2);
  float part_denom = 0.f;
  for (int s = tid; s < num_splits; s += 256) {
    const float l = s == tid ? l_mine : ml[s * 2 + 1];
    const float w = l > 0.f ? exp2f((s == tid ? m_mine : ml[s * 2]) - big) : 0.f;  // an empty split has no weight
    wgt[s] = w;
    part_denom += w * l;
  }
  part_denom = wave_sum(part_denom);
  if (lane == 0) red_sum[wave] = part_denom;
  __syncthreads();
  const float denom = (red_sum[0] + red_sum[1]) + (red_sum[2] + red_sum[3]) + (sink ? exp2f(s2 - big) : 0.f);
  const float inv = denom > 0.f ? 1.f / denom : 0.f;
  if (quads_ok) {
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    if (grp < groups) {
#pragma unroll
      for (int i = 0; i < EARLY; ++i) {
        const int sp = grp + i * groups;
        const float w = sp < num_splits ? wgt[sp] : 0.f;
        a.x = fmaf(w, early[i].x, a.x), a.y = fmaf(w, early[i].y, a.y), a.z = fmaf(w, early[i].z, a.z), a.w = fmaf(w, early[i].w, a.w);
      }
      for (int sp = grp + EARLY * groups; sp < num_splits; sp += groups) {
        const float w = wgt[sp];
        const float4 v = *reinterpret_cast<const float4*>(po + (size_t)sp * dk + qd * 4);
        a.x = fmaf(w, v.x, a.x), a.y = fmaf(w, v.y, a.y), a.z = fmaf(w, v.z, a.z), a.w = fmaf(w, v.w, a.w);
      }
    }
    partial[tid] = a;
    __syncthreads();
    if (tid < quads) {
      float4 total = partial[tid];
      for (int gi = 1; gi < groups; ++gi) {
        const float4 v = partial[gi * quads + tid];
        total.x += v.x, total.y += v.y, total.z += v.z, total.w += v.w;
      }
      lat[4 * tid] = to_float(from_float<bf16_t>(total.x * inv));
      lat[4 * tid + 1] = to_float(from_float<bf16_t>(total.y * inv));
      lat[4 * tid + 2] = to_float(from_float<bf16_t>(total.z * inv));
      lat[4 * tid + 3] = to_float(from_float<bf16_t>(total.w * inv));
#pragma unroll
      for (int i = 0; i < 4; ++i) latb[4 * tid + i] = from_float<bf16_t>(lat[4 * tid + i]);
    }
  } else {
    for (int c = tid; c < rank; c += 256) {
      float a0 = 0.f;
      for (int s = 0; s < num_splits; ++s) a0 = fmaf(wgt[s], po[(size_t)s * dk + c], a0);
      latb[c] = from_float<bf16_t>(a0 * inv);
      lat[c] = to_float(latb[c]);
    }
  }
  __syncthreads();
  const float gv = gate ? 1.f / (1.f + expf(-gate_raw)) : 1.f;
  if (wide) {
    for (int n0 = wave * 16; n0 < dv; n0 += 64) {
      const bf16_t* w = n0 + rr < dv ? W_uv + ((size_t)head * dv + n0 + rr) * rank : nullptr;
      tp_float4 acc = {0.f, 0.f, 0.f, 0.f};
      int k0 = 0;
      if (n0 == wave * 16) {  // the wave's first tile: its first weights were asked for at the kernel's head
#pragma unroll
        for (int i = 0; i < EARLY; ++i) {
          const int at = 32 * i + 8 * gg;
          if (32 * i < rank) {
            tp_bf16x8 xf = tp_bf16x8{};
            if (rr == 0 && at < rank) xf = *reinterpret_cast<const tp_bf16x8*>(latb + at);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wpre[i], xf, acc, 0, 0, 0);
          }
        }
        k0 = 32 * EARLY;
      }
      for (; k0 < rank; k0 += 32) {
        const int at = k0 + 8 * gg;
        tp_bf16x8 wf = tp_bf16x8{}, xf = tp_bf16x8{};
        if (w && at < rank) wf = *reinterpret_cast<const tp_bf16x8*>(w + at);
        if (rr == 0 && at < rank) xf = *reinterpret_cast<const tp_bf16x8*>(latb + at);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf, acc, 0, 0, 0);
      }
      if (rr == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n0 + 4 * gg + i < dv) out[unit * dv + n0 + 4 * gg + i] = from_float<bf16_t>(acc[i] * gv);
      }
    }
  } else {
    for (int j = tid; j < dv; j += 256) {
      const bf16_t* w = W_uv + ((size_t)head * dv + j) * rank;
      float acc = 0.f;
      for (int c = 0; c < rank; ++c) acc = fmaf(to_float(w[c]), lat[c], acc);
      out[unit * dv + j] = from_float<bf16_t>(acc * gv);
    }
  }
}

extern "C" int me_latent_values_supported(int num_splits, int rank) { return num_splits <= LV_MAX_SPLITS && rank <= LV_MAX_RANK; }

extern "C" int me_latent_values_bf16(const float* part_o, const float* part_ml, int num_splits, int dk, int rank, const float* sink,
                                     const void* W_uv, const void* gate, long long gate_row, void* out, int items, int nh, int dv,
                                     hipStream_t stream) {
  if (items <= 0) return 0;
  if (!me_latent_values_supported(num_splits, rank) || num_splits < 1 || rank > dk || nh <= 0 || dv <= 0)
    return me_fail("me_latent_values: splits=%d rank=%d dk=%d heads=%d dv=%d", num_splits, rank, dk, nh, dv);
  latent_values_kernel<<<(unsigned)(items * nh), 256, 0, stream>>>(part_o, part_ml, num_splits, dk, rank, sink, (const bf16_t*)W_uv,
                                                                   (const bf16_t*)gate, (size_t)gate_row, (bf16_t*)out, nh, dv);
  return me_check_launch("me_latent_values");
}
