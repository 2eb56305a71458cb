// The two products of routed experts for prompt-sized steps, on the matrix cores with both operands staged through LDS:
// the tiled product of gemm_mfma.hip over a list of row tiles that each belong to one expert.
//
// A tile is up to BM pairs (token, pick) of one expert, consecutive in the sorted order (routed_ff.hip: plan = number of
// tiles, then expert, first position and pairs of every tile; sorted = the pair at each position). A block owns a tile
// and BN rows of that expert's weight.
//   GATED:  the rows of x are gathered by the pairs' tokens; the BN weight rows are BN/2 gate rows and the BN/2 up rows of
//           the same columns; act(gate) * up goes to acts [position, N].
//   else:   the rows are those of acts; weight * product goes to parts [pick, token, N] in float32, the place the
//           add of the residual stream reads a token's picks from.
// LDS layout, loads (global_load_lds_dwordx4 with the XOR swizzle of the 16-byte pieces), the double-buffered loop over k
// and the fragment reads are those of gemm_tiled_kernel; k is a multiple of 64 and every row 16-byte aligned. Rows past
// a tile's pairs are clamped to its last pair (their products are never stored). A row's sums do not depend on the tile
// it falls into.
#include "common.h"

typedef __bf16 gg_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 gg_bf16x4 __attribute__((ext_vector_type(4)));
typedef float gg_float4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void* gg_global_ptr;
typedef __attribute__((address_space(3))) void* gg_lds_ptr;

namespace {
constexpr int GGK = 64;  // k per LDS tile; also the LDS row length in elements

// MODE 0: the down product; 1: gate and up rows; 2: up rows alone (experts without a gate: act(x_e . Wu_e^T) -> acts).
template <int BM, int BN, int WM, int WN, int MODE>
__global__ __launch_bounds__(WM * WN * 64) void gemm_grouped_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                     const int* __restrict__ plan, const int* __restrict__ sorted,
                                                                     const float* __restrict__ wts, bf16_t* __restrict__ acts,
                                                                     float* __restrict__ parts, int num_tokens, int N, int K,
                                                                     int top, int n_tiles, int gate, float limit) {
  constexpr bool GATED = MODE == 1, GATHER = MODE != 0;
  constexpr int THREADS = WM * WN * 64;
  constexpr int WMR = BM / WM, WNR = BN / WN;
  constexpr int FM = WMR / 16, FN = WNR / 16;
  constexpr int NX = BM * 8 / THREADS, NW = BN * 8 / THREADS;
  static_assert(WMR % 16 == 0 && WNR % 16 == 0 && BM * 8 % THREADS == 0 && BN * 8 % THREADS == 0, "tile shape");
  static_assert(!GATED || FN % 2 == 0, "a wave needs gate and up fragments in pairs");
  constexpr int COLS = GATED ? BN / 2 : BN;
  extern __shared__ __align__(16) unsigned char gg_lds[];
  bf16_t* sx = reinterpret_cast<bf16_t*>(gg_lds);  // [2][BM][GGK]
  bf16_t* sw = sx + 2 * BM * GGK;                  // [2][BN][GGK]

  const int ti = blockIdx.x / n_tiles, tn = blockIdx.x - ti * n_tiles;  // the blocks of a tile side by side: they share its rows
  if (ti >= plan[0]) return;
  const int e = plan[1 + 3 * ti], begin = plan[2 + 3 * ti], rows = plan[3 + 3 * ti];
  const int n0 = tn * COLS;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave % WM, wn = wave / WM;
  const int r = lane & 15, g = lane >> 4;

  const bf16_t* px[NX];
  const bf16_t* pw[NW];
#pragma unroll
  for (int i = 0; i < NX; ++i) {
    const int tr = (tid + i * THREADS) >> 3;
    const int at = begin + min(tr, rows - 1);
    const size_t row = GATHER ? (size_t)(sorted[at] / top) : (size_t)at;
    px[i] = X + row * K + (((tid & 7) ^ ((tr >> 1) & 7)) * 8);
  }
  const int w_rows = GATED ? 2 * N : N;
  const bf16_t* We = W + (size_t)e * w_rows * K;
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int tr = (tid + i * THREADS) >> 3;
    int row = n0 + tr;
    if (GATED) {
      const int w = tr / WNR, q = tr % WNR;
      row = min(n0 + w * (WNR / 2) + q % (WNR / 2), N - 1) + (q >= WNR / 2 ? N : 0);
    }
    pw[i] = We + (size_t)min(row, w_rows - 1) * K + (((tid & 7) ^ ((tr >> 1) & 7)) * 8);
  }
  auto request = [&](int k, int b) {
    char* dx = reinterpret_cast<char*>(sx + b * BM * GGK) + wave * 1024;
    char* dw = reinterpret_cast<char*>(sw + b * BN * GGK) + wave * 1024;
#pragma unroll
    for (int i = 0; i < NX; ++i)
      __builtin_amdgcn_global_load_lds((gg_global_ptr)(px[i] + k), (gg_lds_ptr)(dx + i * THREADS * 16), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < NW; ++i)
      __builtin_amdgcn_global_load_lds((gg_global_ptr)(pw[i] + k), (gg_lds_ptr)(dw + i * THREADS * 16), 16, 0, 0);
  };

  gg_float4 acc[FN][FM];
#pragma unroll
  for (int a = 0; a < FN; ++a)
#pragma unroll
    for (int b = 0; b < FM; ++b) acc[a][b] = (gg_float4){0.f, 0.f, 0.f, 0.f};

  const int steps = K / GGK;
  request(0, 0);
  __syncthreads();
  const int frag_x = (wm * WMR + r) * GGK, frag_w = (wn * WNR + r) * GGK;
  const int piece[2] = {(g ^ ((r >> 1) & 7)) * 8, ((4 + g) ^ ((r >> 1) & 7)) * 8};
  for (int s = 0; s < steps; ++s) {
    const int cur = s & 1;
    const bf16_t* cx = sx + cur * BM * GGK + frag_x;
    const bf16_t* cw = sw + cur * BN * GGK + frag_w;
    request(min(s + 1, steps - 1) * GGK, cur ^ 1);
#pragma unroll
    for (int kk = 0; kk < GGK / 32; ++kk) {
      gg_bf16x8 fx[FM], fw[FN];
#pragma unroll
      for (int b = 0; b < FM; ++b) fx[b] = *reinterpret_cast<const gg_bf16x8*>(cx + b * 16 * GGK + piece[kk]);
#pragma unroll
      for (int a = 0; a < FN; ++a) fw[a] = *reinterpret_cast<const gg_bf16x8*>(cw + a * 16 * GGK + piece[kk]);
#pragma unroll
      for (int a = 0; a < FN; ++a)
#pragma unroll
        for (int b = 0; b < FM; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[a], fx[b], acc[a][b], 0, 0, 0);
    }
    __syncthreads();
  }

  // lane holds C[row of the tile = .. + r][n = .. + 4 g + i]
#pragma unroll
  for (int b = 0; b < FM; ++b) {
    const int m = wm * WMR + b * 16 + r;
    if (m >= rows) continue;
    if constexpr (GATED) {
#pragma unroll
      for (int a = 0; a < FN / 2; ++a) {
        const int n = n0 + wn * (WNR / 2) + a * 16 + 4 * g;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          v[i] = gate == ME_GATE_CLAMPED_SIGMOID ? gated_pair(acc[a][b][i], acc[a + FN / 2][b][i], gate, limit)
                                                 : gate_act_bf16(acc[a][b][i], gate) * acc[a + FN / 2][b][i];
        bf16_t* p = acts + (size_t)(begin + m) * N + n;
        if (n + 3 < N && (((uintptr_t)p) & 7) == 0) {
          const gg_bf16x4 w = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
          *reinterpret_cast<gg_bf16x4*>(p) = w;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) p[i] = from_float<bf16_t>(v[i]);
        }
      }
    } else if constexpr (GATHER) {
#pragma unroll
      for (int a = 0; a < FN; ++a) {
        const int n = n0 + wn * WNR + a * 16 + 4 * g;
        bf16_t* p = acts + (size_t)(begin + m) * N + n;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) p[i] = from_float<bf16_t>(ungated_act(acc[a][b][i], gate));
      }
    } else {
      const int pair = sorted[begin + m];
      const float wgt = wts[pair];
      float* prow = parts + ((size_t)(pair % top) * num_tokens + pair / top) * N;
#pragma unroll
      for (int a = 0; a < FN; ++a) {
        const int n = n0 + wn * WNR + a * 16 + 4 * g;
        if (n + 3 < N && (((uintptr_t)(prow + n)) & 15) == 0) {
          *reinterpret_cast<float4*>(prow + n) = make_float4(wgt * acc[a][b][0], wgt * acc[a][b][1], wgt * acc[a][b][2], wgt * acc[a][b][3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) prow[n + i] = wgt * acc[a][b][i];
        }
      }
    }
  }
}

template <int MODE>
int launch_grouped(const bf16_t* X, const bf16_t* W, const int* plan, const int* sorted, const float* wts, bf16_t* acts, float* parts,
                   int num_tokens, int N, int K, int top, int max_tiles, int gate, float limit, hipStream_t stream) {
  constexpr int BM = 128, BN = 128, WM = 4, WN = 2;
  constexpr int COLS = MODE == 1 ? BN / 2 : BN;
  constexpr size_t LDS = (size_t)2 * (BM + BN) * GGK * sizeof(bf16_t);
  auto kernel = gemm_grouped_kernel<BM, BN, WM, WN, MODE>;
  static bool raised = false;
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS) != hipSuccess)
      return me_fail("me_gemm_grouped: %zu bytes of LDS were refused", LDS);
    raised = true;
  }
  const int n_tiles = (N + COLS - 1) / COLS;
  if ((long long)max_tiles * n_tiles > 0x7fffffffLL) return me_fail("me_gemm_grouped: %d x %d blocks exceed the grid", max_tiles, n_tiles);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(max_tiles * n_tiles)), dim3(WM * WN * 64), LDS, stream, X, W, plan, sorted, wts, acts, parts,
                     num_tokens, N, K, top, n_tiles, gate, limit);
  return me_check_launch("me_gemm_grouped");
}
}  // namespace

// Rows a tile of the list holds for these kernels.
extern "C" int me_gemm_grouped_tile_rows() { return 128; }

// gated != 0: acts [P, N] = act(x_e . Wg_e^T) * (x_e . Wu_e^T), x rows gathered by token (W [E, 2 N, K]); else
// (limit: what the activations with a limit clamp by)
// parts [top, tokens, N] = weight * (acts_e . Wd_e^T) (W [E, N, K], X = acts [P, K]). max_tiles: an upper bound of the list's length.
extern "C" int me_gemm_grouped_bf16(const void* X, const void* W, const int* plan, const int* sorted, const float* wts, void* acts,
                                    float* parts, int num_tokens, int N, int K, int top, int max_tiles, int gated, float limit,
                                    hipStream_t stream) {
  if (num_tokens <= 0 || max_tiles <= 0) return 0;
  if (K <= 0 || K % GGK) return me_fail("me_gemm_grouped: K=%d must be a positive multiple of %d", K, GGK);
  if (((uintptr_t)X | (uintptr_t)W) & 15) return me_fail("me_gemm_grouped: operands must be 16-byte aligned");
  if (act_is_ungated(gated))  // an activation without a gate: W [E, N, K], acts [P, N] = act(x_e . W_e^T), x rows gathered by token
    return launch_grouped<2>((const bf16_t*)X, (const bf16_t*)W, plan, sorted, wts, (bf16_t*)acts, nullptr, num_tokens, N, K, top,
                             max_tiles, gated, limit, stream);
  if (gated)
    return launch_grouped<1>((const bf16_t*)X, (const bf16_t*)W, plan, sorted, wts, (bf16_t*)acts, nullptr, num_tokens, N, K, top,
                                max_tiles, gated, limit, stream);
  return launch_grouped<0>((const bf16_t*)X, (const bf16_t*)W, plan, sorted, wts, nullptr, parts, num_tokens, N, K, top, max_tiles, 0,
                               0.f, stream);
}
