// Linear attention with a decay per token, head and key channel and a bonus for the current token (the time mixing of RWKV-6),
// a d x d float32 state per request and head:
//
//     o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,        S_t = diag(w_t) S_(t-1) + k_t v_t^T
//
// Every projection reads a blend of the token's input and the input of the token before it, h + (h' - h) * mu, with a mu of its own.
//
//   shift    for every token the five blends (r, k, v, gate, decay) in the activations' type; h' of an item's first token is the
//            item's state row (zeros at position 0). A second launch keeps the item's last input as the next h'.
//   decay    w = exp(-exp(W_2 tanh(z) + w_0)) in float32 for all tokens, z the decay's inner projection.
//   scan     a wave per (item, head, 4 value channels): a row of 16 lanes a column of S, each lane d / 16 of the column's rows in
//            registers; the wave walks the item's tokens, and a column's sum over its row of lanes is four data-parallel moves.
//            Sums run in an order that the head's size alone fixes (a lane's rows in ascending order, then the row of lanes
//            pairwise), in both forms of the kernel: a token's result is the same bits however the sequence was cut and whatever
//            else the step holds.
//   finish   every head's o over its root mean square, times a weight, times silu(gate), times the caller's scale.
//
// State row of a slot: [heads, d (key), d (value)] float32, then the `width` elements of h'.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void time_shift_kernel(const T* __restrict__ h, const float* __restrict__ state, long long state_row,
                                                         long long prev_at, const int* __restrict__ state_slots,
                                                         const int* __restrict__ item_start, const int* __restrict__ token_item,
                                                         const int* __restrict__ positions, const float* __restrict__ mu,
                                                         T* __restrict__ o0, T* __restrict__ o1, T* __restrict__ o2, T* __restrict__ o3,
                                                         T* __restrict__ o4, int width, long long out_stride) {
  const int t = blockIdx.x, item = token_item[t];
  const bool from_state = t == item_start[item];
  const float* prev_row = state + (size_t)state_slots[item] * state_row + prev_at;
  const bool none = positions[t] == 0;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float x = to_float(h[(size_t)t * width + i]);
    const float prev = none ? 0.f : (from_state ? prev_row[i] : to_float(h[(size_t)(t - 1) * width + i]));
    const float dlt = prev - x;
    const size_t at = (size_t)t * out_stride + i;  // (the blends' rows may lie interleaved in one buffer)
    o0[at] = from_float<T>(fmaf(dlt, mu[i], x));
    o1[at] = from_float<T>(fmaf(dlt, mu[width + i], x));
    o2[at] = from_float<T>(fmaf(dlt, mu[2 * width + i], x));
    o3[at] = from_float<T>(fmaf(dlt, mu[3 * width + i], x));
    o4[at] = from_float<T>(fmaf(dlt, mu[4 * width + i], x));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void time_shift_keep_kernel(const T* __restrict__ h, float* __restrict__ state, long long state_row,
                                                              long long prev_at, const int* __restrict__ state_slots,
                                                              const int* __restrict__ item_start, int width) {
  const int item = blockIdx.x, last = item_start[item + 1] - 1;
  if (last < item_start[item]) return;
  float* prev_row = state + (size_t)state_slots[item] * state_row + prev_at;
  for (int i = threadIdx.x; i < width; i += blockDim.x) prev_row[i] = to_float(h[(size_t)last * width + i]);
}

// h [T, width]; mu float32 [5, width] (r, k, v, gate, decay); outs: five buffers in the activations' type whose rows of `width` elements
// lie out_stride elements apart (width: five plain [T, width] buffers; 5 * width and bases a row apart: one buffer [T, 5, width]).
extern "C" int me_time_shift(const void* h, float* state, long long state_row, long long prev_at, const int* state_slots,
                             const int* item_start, const int* token_item, const int* positions, const float* mu, void* const* outs,
                             long long out_stride, int num_tokens, int items, int width, int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (width <= 0 || prev_at < 0 || prev_at + width > state_row) return me_fail("me_time_shift: width=%d at %lld of a row of %lld", width, prev_at, state_row);
  if (dtype == ME_F32) {
    time_shift_kernel<float><<<num_tokens, 256, 0, stream>>>((const float*)h, state, state_row, prev_at, state_slots, item_start, token_item,
                                                             positions, mu, (float*)outs[0], (float*)outs[1], (float*)outs[2],
                                                             (float*)outs[3], (float*)outs[4], width, out_stride);
    time_shift_keep_kernel<float><<<items, 256, 0, stream>>>((const float*)h, state, state_row, prev_at, state_slots, item_start, width);
  } else {
    time_shift_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>((const bf16_t*)h, state, state_row, prev_at, state_slots, item_start,
                                                              token_item, positions, mu, (bf16_t*)outs[0], (bf16_t*)outs[1],
                                                              (bf16_t*)outs[2], (bf16_t*)outs[3], (bf16_t*)outs[4], width, out_stride);
    time_shift_keep_kernel<bf16_t><<<items, 256, 0, stream>>>((const bf16_t*)h, state, state_row, prev_at, state_slots, item_start, width);
  }
  return me_check_launch("me_time_shift");
}

#define TM_MAX_RANK 1024

// A column's sum over its row of 16 lanes (the lanes of a wave whose numbers differ in their low four bits), in every lane of the
// row, by four data-parallel moves (no LDS): a rotation by 8, one by 4, then the two exchanges inside a group of four add the same
// pairs in every lane, so all lanes hold the same bits.
__device__ __forceinline__ float row16_sum(float x) {
#define TM_DPP_ADD(CTRL) x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false))
  TM_DPP_ADD(0x128);  // row_ror:8
  TM_DPP_ADD(0x124);  // row_ror:4
  TM_DPP_ADD(0x4e);   // quad_perm:[2,3,0,1]
  TM_DPP_ADD(0xb1);   // quad_perm:[1,0,3,2]
#undef TM_DPP_ADD
  return x;
}

// A wave per (item, head, group of 4 value channels); RPL: rows of S a lane holds (d <= 16 * RPL). Lane l: column 4 * group + l / 16,
// rows (l % 16) * per .. + per - 1 with per = ceil(d / 16).
template <typename T, int RPL>
__global__ __launch_bounds__(64) void time_scan_kernel(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
                                                       const float* __restrict__ decay, const float* __restrict__ bonus,
                                                       float* __restrict__ state, long long state_row, const int* __restrict__ state_slots,
                                                       const int* __restrict__ item_start, float* __restrict__ o, int heads, int d,
                                                       long long in_stride) {
  const int groups = (d + 3) / 4;
  const int item = blockIdx.x / (heads * groups), head = (blockIdx.x / groups) % heads, grp = blockIdx.x % groups;
  const int lane = threadIdx.x, rp = lane & 15, c = grp * 4 + (lane >> 4);
  const int per = (d + 15) / 16, i0 = rp * per;
  const int first = item_start[item], end = item_start[item + 1];
  const bool col = c < d;
  const int n = heads * d;
  float* S = state + (size_t)state_slots[item] * state_row + (size_t)head * d * d;
  float s[RPL], u[RPL];
#pragma unroll
  for (int a = 0; a < RPL; ++a) {
    const int i = i0 + a;
    const bool there = a < per && i < d;
    s[a] = there && col ? S[(size_t)i * d + c] : 0.f;
    u[a] = there ? bonus[head * d + i] : 0.f;
  }
  for (int t = first; t < end; ++t) {
    const size_t at = (size_t)t * n + head * d, in = (size_t)t * in_stride + head * d;  // (rows of r, k, v may be wider than n)
    const float vc = col ? to_float(v[in + c]) : 0.f;
    float rr[RPL], kk[RPL], ww[RPL];
#pragma unroll
    for (int a = 0; a < RPL; ++a) {
      const int i = i0 + a;
      const bool there = a < per && i < d;
      rr[a] = there ? to_float(r[in + i]) : 0.f;
      kk[a] = there ? to_float(k[in + i]) : 0.f;
      ww[a] = there ? decay[at + i] : 0.f;
    }
    float acc = 0.f;
#pragma unroll
    for (int a = 0; a < RPL; ++a) {
      const float kv = kk[a] * vc;
      acc = fmaf(rr[a], fmaf(u[a], kv, s[a]), acc);
      s[a] = fmaf(ww[a], s[a], kv);
    }
    acc = row16_sum(acc);
    if (rp == 0 && col) o[at + c] = acc;
  }
#pragma unroll
  for (int a = 0; a < RPL; ++a) {
    const int i = i0 + a;
    if (a < per && i < d && col) S[(size_t)i * d + c] = s[a];
  }
}

// The scan for heads of D = 32, 64 or 128 elements, a block of four waves per (item, head, 16 value channels), a wave per 4 of them. The
// block walks the item's tokens in chunks of TS_CHUNK (half as many for heads of 128): all threads fetch a chunk's r, k and decays (the head's whole rows) and the v of
// the block's channels together (16 bytes a load, every load of the chunk in flight at once, and the next chunk's asked for before
// this one is worked on) and lay them out in LDS as float32; then every wave walks the chunk's tokens out of LDS. The sums are those
// of time_scan_kernel, in its order: a token's result is the same bits whichever of the two kernels serves it.
#define TS_CHUNK 32
template <typename T>
struct TsVec;  // eight consecutive elements of a row
template <>
struct TsVec<bf16_t> {
  uint4 raw;
  __device__ __forceinline__ void load(const bf16_t* p) { raw = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void zero() { raw = make_uint4(0, 0, 0, 0); }
  __device__ __forceinline__ void store(float* dst) const {
    const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dst[2 * i] = __uint_as_float(w4[i] << 16);
      dst[2 * i + 1] = __uint_as_float(w4[i] & 0xffff0000u);
    }
  }
};
template <>
struct TsVec<float> {
  float4 a, b;
  __device__ __forceinline__ void load(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ __forceinline__ void zero() { a = b = make_float4(0.f, 0.f, 0.f, 0.f); }
  __device__ __forceinline__ void store(float* dst) const {
    *reinterpret_cast<float4*>(dst) = a;
    *reinterpret_cast<float4*>(dst + 4) = b;
  }
};

// decay[t, c] = exp(-exp(sum_j W2[c, j] tanh(z[t, j]) + w0[c])). Grid (runs of TD_TOKENS tokens, runs of 256 channels), a thread a
// channel: it walks its row of W2 eight elements a load and meets every token of the run with each piece, so that a row is fetched
// once for the run's tokens. The sum over j runs in ascending j for every token, whatever else the step holds.
#define TD_TOKENS 8
template <typename T>
__global__ __launch_bounds__(256) void time_decay_kernel(const T* __restrict__ z, const T* __restrict__ W2, const float* __restrict__ w0,
                                                         float* __restrict__ decay, int num_tokens, int n, int rank, long long z_stride) {
  extern __shared__ float th[];  // [TD_TOKENS][rank]
  const int t0 = blockIdx.x * TD_TOKENS, count = min(TD_TOKENS, num_tokens - t0);
  for (int i = threadIdx.x; i < count * rank; i += blockDim.x) th[i] = tanhf(to_float(z[(size_t)(t0 + i / rank) * z_stride + i % rank]));
  __syncthreads();
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const T* wr = W2 + (size_t)c * rank;
  float sum[TD_TOKENS];
#pragma unroll
  for (int k = 0; k < TD_TOKENS; ++k) sum[k] = 0.f;
  const bool vec = rank % 8 == 0 && (((uintptr_t)W2) & 15) == 0;
  int j = 0;
  if (vec)
    for (; j + 8 <= rank; j += 8) {
      TsVec<T> piece;
      piece.load(wr + j);
      __attribute__((aligned(16))) float w8[8];
      piece.store(w8);
#pragma unroll
      for (int k = 0; k < TD_TOKENS; ++k)
        if (k < count) {
#pragma unroll
          for (int i = 0; i < 8; ++i) sum[k] = fmaf(w8[i], th[k * rank + j + i], sum[k]);
        }
    }
  for (; j < rank; ++j) {
    const float w = to_float(wr[j]);
#pragma unroll
    for (int k = 0; k < TD_TOKENS; ++k)
      if (k < count) sum[k] = fmaf(w, th[k * rank + j], sum[k]);
  }
  const float bias = w0[c];
#pragma unroll
  for (int k = 0; k < TD_TOKENS; ++k)
    if (k < count) decay[(size_t)(t0 + k) * n + c] = expf(-expf(sum[k] + bias));
}

template <typename T, int D>
__global__ __launch_bounds__(256) void time_scan_chunked_kernel(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
                                                                const float* __restrict__ decay, const float* __restrict__ bonus,
                                                                float* __restrict__ state, long long state_row,
                                                                const int* __restrict__ state_slots, const int* __restrict__ item_start,
                                                                float* __restrict__ o, int heads) {
  constexpr int RPL = D / 16, VPR = D / 8;       // rows of S a lane holds; vectors of eight elements a row
  constexpr int CH = D > 64 ? TS_CHUNK / 2 : TS_CHUNK;  // tokens a chunk: a thread fetches one vector of each array
  constexpr int NV = (CH * VPR + 255) / 256;  // vectors of a chunk's r (k, decays) a thread fetches
  constexpr int PARTS = D / 16;                  // blocks a head
  __shared__ __attribute__((aligned(16))) float lr[CH][D], lk[CH][D], lw[CH][D], lv[CH][16];
  const int item = blockIdx.x / (heads * PARTS), head = (blockIdx.x / PARTS) % heads, part = blockIdx.x % PARTS;
  const int tid = threadIdx.x, wave = tid / ME_WAVE, lane = tid & (ME_WAVE - 1);
  const int rp = lane & 15, cl = wave * 4 + (lane >> 4), c = part * 16 + cl, i0 = rp * RPL;
  const int first = item_start[item], end = item_start[item + 1];
  const int n = heads * D;
  float* S = state + (size_t)state_slots[item] * state_row + (size_t)head * D * D;
  float s[RPL], u[RPL];
#pragma unroll
  for (int a = 0; a < RPL; ++a) {
    s[a] = S[(size_t)(i0 + a) * D + c];
    u[a] = bonus[head * D + i0 + a];
  }
  TsVec<T> fr[NV], fk[NV], fv;
  float4 fw0[NV], fw1[NV];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const int vi = tid + 256 * q, t = t0 + vi / VPR, ve = 8 * (vi % VPR);
      if (vi < CH * VPR && t < end) {
        const size_t at = (size_t)t * n + head * D + ve;
        fr[q].load(r + at);
        fk[q].load(k + at);
        fw0[q] = *reinterpret_cast<const float4*>(decay + at);
        fw1[q] = *reinterpret_cast<const float4*>(decay + at + 4);
      } else {
        fr[q].zero(), fk[q].zero();
        fw0[q] = fw1[q] = make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
    fv.zero();
    if (tid < CH * 2 && t0 + tid / 2 < end)  // the block's 16 value channels: two vectors a token
      fv.load(v + (size_t)(t0 + tid / 2) * n + head * D + part * 16 + 8 * (tid % 2));
  };
  if (first < end) fetch(first);
  for (int t0 = first; t0 < end; t0 += CH) {
    __syncthreads();  // the chunk before is worked off
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const int vi = tid + 256 * q, vt = vi / VPR, ve = 8 * (vi % VPR);
      if (vi < CH * VPR) {
        fr[q].store(&lr[vt][ve]);
        fk[q].store(&lk[vt][ve]);
        *reinterpret_cast<float4*>(&lw[vt][ve]) = fw0[q];
        *reinterpret_cast<float4*>(&lw[vt][ve + 4]) = fw1[q];
      }
    }
    if (tid < CH * 2) fv.store(&lv[tid / 2][8 * (tid % 2)]);
    __syncthreads();
    if (t0 + CH < end) fetch(t0 + CH);  // on its way while this chunk is worked on
    const int count = min(CH, end - t0);
    auto token = [&](int j) {
      const float vc = lv[j][cl];
      float rr[RPL], kk[RPL], ww[RPL];
      if constexpr (RPL % 4 == 0) {
#pragma unroll
        for (int a4 = 0; a4 < RPL / 4; ++a4) {
          const float4 r4 = *reinterpret_cast<const float4*>(&lr[j][i0 + 4 * a4]);
          const float4 k4 = *reinterpret_cast<const float4*>(&lk[j][i0 + 4 * a4]);
          const float4 w4 = *reinterpret_cast<const float4*>(&lw[j][i0 + 4 * a4]);
          rr[4 * a4] = r4.x, rr[4 * a4 + 1] = r4.y, rr[4 * a4 + 2] = r4.z, rr[4 * a4 + 3] = r4.w;
          kk[4 * a4] = k4.x, kk[4 * a4 + 1] = k4.y, kk[4 * a4 + 2] = k4.z, kk[4 * a4 + 3] = k4.w;
          ww[4 * a4] = w4.x, ww[4 * a4 + 1] = w4.y, ww[4 * a4 + 2] = w4.z, ww[4 * a4 + 3] = w4.w;
        }
      } else {
#pragma unroll
        for (int a = 0; a < RPL; ++a) rr[a] = lr[j][i0 + a], kk[a] = lk[j][i0 + a], ww[a] = lw[j][i0 + a];
      }
      float acc = 0.f;
#pragma unroll
      for (int a = 0; a < RPL; ++a) {
        const float kv = kk[a] * vc;
        acc = fmaf(rr[a], fmaf(u[a], kv, s[a]), acc);
        s[a] = fmaf(ww[a], s[a], kv);
      }
      acc = row16_sum(acc);
      if (rp == 0) o[(size_t)(t0 + j) * n + head * D + c] = acc;
    };
    // four tokens a turn without a branch between them: a token's sum over the row of lanes and its store run under the next tokens'
    // multiply-adds (only the state's way from token to token, one multiply-add a row, is in order)
    int j = 0;
    for (; j + 4 <= count; j += 4) {
      token(j);
      token(j + 1);
      token(j + 2);
      token(j + 3);
    }
    for (; j < count; ++j) token(j);
  }
#pragma unroll
  for (int a = 0; a < RPL; ++a) S[(size_t)(i0 + a) * D + c] = s[a];
}

// A wave per (token, head): o over its root mean square, times the weight, silu(gate) and the scale, into out at column out_col.
template <typename T>
__global__ __launch_bounds__(256) void time_finish_kernel(const float* __restrict__ o, const T* __restrict__ gate, const float* __restrict__ w,
                                                          T* __restrict__ out, long long out_row, int out_col, float out_scale,
                                                          long long units, int heads, int d, float eps, long long in_stride) {
  const long long unit = (long long)blockIdx.x * (blockDim.x / ME_WAVE) + threadIdx.x / ME_WAVE;
  if (unit >= units) return;
  const int lane = threadIdx.x & (ME_WAVE - 1);
  const long long t = unit / heads;
  const int head = (int)(unit % heads), n = heads * d;
  const float* orow = o + (size_t)t * n + head * d;
  float ss = 0.f;
  for (int i = lane; i < d; i += ME_WAVE) ss = fmaf(orow[i], orow[i], ss);
  const float rinv = rsqrtf(wave_sum(ss) / (float)d + eps) * out_scale;
  for (int i = lane; i < d; i += ME_WAVE) {
    const float g = to_float(gate[(size_t)t * in_stride + head * d + i]);
    out[(size_t)t * out_row + out_col + head * d + i] = from_float<T>(orow[i] * rinv * w[head * d + i] * (g / (1.f + expf(-g))));
  }
}

extern "C" long long me_time_mix_workspace(long long tokens, int heads, int d) { return 2 * tokens * heads * d * 4 + 512; }

// r, k, v, gate (rows of heads * d elements) and z (rows of rank) in the activations' type, their rows in_stride elements apart (0:
// plain [T, heads * d] and [T, rank] buffers); W2 [heads * d, rank] in the activations' type; w0, bonus,
// norm_w float32 [heads * d]; state float32 rows of state_row elements whose first heads * d * d are S. out [T, out_row], the
// result at column out_col. workspace: me_time_mix_workspace bytes.
extern "C" int me_time_mix(const void* r, const void* k, const void* v, const void* gate, const void* z, const void* W2, const float* w0,
                           const float* bonus, const float* norm_w, float* state, long long state_row, const int* state_slots,
                           const int* item_start, void* out, long long out_row, int out_col, float out_scale, int num_tokens, int items,
                           int heads, int d, int rank, float eps, long long in_stride, int dtype, void* workspace, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (heads <= 0 || d <= 0 || d > 256) return me_fail("me_time_mix: %d heads of %d elements (at most 256)", heads, d);
  if (rank <= 0 || rank > TM_MAX_RANK) return me_fail("me_time_mix: a decay of inner size %d (at most %d)", rank, TM_MAX_RANK);
  const long long n = (long long)heads * d;
  if (out_col < 0 || out_col + n > out_row) return me_fail("me_time_mix: the result at column %d of a row of %lld", out_col, out_row);
  if ((long long)heads * d * d > state_row) return me_fail("me_time_mix: state rows of %lld elements", state_row);
  float* decay = (float*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  float* o = decay + (size_t)num_tokens * n;
  const unsigned scan_blocks = (unsigned)(items * heads * ((d + 3) / 4));
  const long long units = (long long)num_tokens * heads;
  const unsigned fin_blocks = (unsigned)((units + 3) / 4);
  // steps that bring an item more than a token or two, heads of 32, 64 or 128 elements, rows at multiples of 16 bytes: the kernel that
  // stages chunks of tokens in LDS
  const long long rows_apart = in_stride > 0 ? in_stride : n, z_apart = in_stride > 0 ? in_stride : rank;
  const bool chunked = in_stride <= 0 && num_tokens >= 4 * items && (d == 32 || d == 64 || d == 128) &&
                       ((((uintptr_t)r | (uintptr_t)k | (uintptr_t)v | (uintptr_t)decay)) & 15) == 0;
#define ME_TM_RUN(TT)                                                                                                               \
  do {                                                                                                                              \
    time_decay_kernel<TT><<<dim3((num_tokens + TD_TOKENS - 1) / TD_TOKENS, (unsigned)((n + 255) / 256)), 256,                       \
                            (size_t)TD_TOKENS * rank * sizeof(float), stream>>>((const TT*)z, (const TT*)W2, w0, decay, num_tokens,  \
                                                                                (int)n, rank, z_apart);                             \
    if (chunked && d == 32)                                                                                                         \
      time_scan_chunked_kernel<TT, 32><<<items * heads * 2, 256, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, decay, bonus, state, \
                                                                          state_row, state_slots, item_start, o, heads);           \
    else if (chunked && d == 64)                                                                                                    \
      time_scan_chunked_kernel<TT, 64><<<items * heads * 4, 256, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, decay, bonus, state, \
                                                                          state_row, state_slots, item_start, o, heads);           \
    else if (chunked && d == 128)                                                                                                   \
      time_scan_chunked_kernel<TT, 128><<<items * heads * 8, 256, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, decay, bonus, state, \
                                                                           state_row, state_slots, item_start, o, heads);          \
    else if (d <= 32)                                                                                                                    \
      time_scan_kernel<TT, 2><<<scan_blocks, 64, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, decay, bonus, state, state_row, \
                                                              state_slots, item_start, o, heads, d, rows_apart);                                \
    else if (d <= 64)                                                                                                               \
      time_scan_kernel<TT, 4><<<scan_blocks, 64, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, decay, bonus, state, state_row, \
                                                               state_slots, item_start, o, heads, d, rows_apart);                               \
    else if (d <= 128)                                                                                                              \
      time_scan_kernel<TT, 8><<<scan_blocks, 64, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, decay, bonus, state, state_row, \
                                                               state_slots, item_start, o, heads, d, rows_apart);                               \
    else                                                                                                                            \
      time_scan_kernel<TT, 16><<<scan_blocks, 64, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, decay, bonus, state, state_row, \
                                                               state_slots, item_start, o, heads, d, rows_apart);                               \
    time_finish_kernel<TT><<<fin_blocks, 256, 0, stream>>>(o, (const TT*)gate, norm_w, (TT*)out, out_row, out_col, out_scale, units,  \
                                                           heads, d, eps, rows_apart);                                                          \
  } while (0)
  if (dtype == ME_F32)
    ME_TM_RUN(float);
  else
    ME_TM_RUN(bf16_t);
#undef ME_TM_RUN
  return me_check_launch("me_time_mix");
}
