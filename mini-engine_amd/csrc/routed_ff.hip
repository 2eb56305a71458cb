// A feed-forward of routed experts: a router picks `top` of E small gated feed-forwards per token and weights them by
// the softmax over the picked logits; the token's result is the weighted sum of what they give.
//
//   route    z = W_r h in float32 (W_r float32), the `top` largest by repeated maximum (the lower index among equals), their
//            weights exp(z_j - z_max) / sum; a (token, rank j) is a *pair*;
//   sort     the pairs grouped by expert (a counting sort in one block), and a list of tiles of up to 16 pairs of one expert;
//   gate/up  per tile: act(W_gate_e h) * (W_up_e h) for the tile's tokens -> acts [pair position, ff];
//   down     per tile: weight * (W_down_e acts) -> parts [j, token, :] in float32: the `top` results of a token lie a
//            stride apart, as partial sums that the next add of the residual stream sums up in the order of j.
// A pair's result does not depend on the tile it falls into (tile_product.h), so a token's result does not depend on
// what else the step holds. Everything stays on the device: a step that a graph replays routes anew every time.
#include "tile_product.h"

extern "C" int me_gemm_grouped_tile_rows();
extern "C" int me_gemm_grouped_bf16(const void* X, const void* W, const int* plan, const int* sorted, const float* wts, void* acts,
                                    float* parts, int num_tokens, int N, int K, int top, int max_tiles, int gated, float limit,
                                    hipStream_t stream);

#define RF_MAX_EXPERTS 1024
#define RF_MAX_TOP 32
#define RF_SCORE_SOFTMAX 0  // the picks' weights: the softmax over the picked logits
#define RF_SCORE_SIGMOID 1  // the picks' scores sigmoid(z) over their sum (+ 1e-20), times a scale; picks bounded by groups
#define RF_SCORE_SOFTMAX_ALL 2  // scores softmax(z) over all router outputs; picked by score + correction; the weights are the picks'
                               // scores as they are, times a scale. The last outputs may stand for identity experts (no tensors:
                               // the token's input itself, times the weight)
#define RF_DIRECT_PAIRS 16  // steps of up to this many pairs (token, pick) are not sorted: a pair is a tile

template <typename T>
__global__ __launch_bounds__(1024) void routed_route_kernel(const T* __restrict__ h, const float* __restrict__ Wr, int* __restrict__ ids,
                                                            float* __restrict__ wts, int hidden, int E, int top,
                                                            int* __restrict__ plan, int* __restrict__ sorted, int num_pairs,
                                                            int scoring, int n_groups, int keep_groups, float route_scale,
                                                            float* __restrict__ shared_gate, int n_identity,
                                                            const float* __restrict__ correction) {
  __shared__ float z[RF_MAX_EXPERTS + 1], sc[RF_MAX_EXPERTS], gs[RF_MAX_EXPERTS];
  const int E_real = E;  // experts that have tensors; the router's outputs E_real .. E - 1 are identity experts
  E += n_identity;
  const int t = blockIdx.x, wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const T* row = h + (size_t)t * hidden;
  // a wave an expert at a time; a lane's elements lie 64 apart, four of them in flight together with sums of their own
  const int waves = blockDim.x / ME_WAVE;
  const int logits = E + (shared_gate ? 1 : 0);  // (the row behind the experts': the gate of an expert that every token uses)
  for (int e = wave; e < logits; e += waves) {
    const float* w = Wr + (size_t)e * hidden;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int c = lane;
    for (; c + 3 * ME_WAVE < hidden; c += 4 * ME_WAVE) {
      const float x0 = to_float(row[c]), x1 = to_float(row[c + ME_WAVE]), x2 = to_float(row[c + 2 * ME_WAVE]),
                  x3 = to_float(row[c + 3 * ME_WAVE]);
      const float w0 = w[c], w1 = w[c + ME_WAVE], w2 = w[c + 2 * ME_WAVE], w3 = w[c + 3 * ME_WAVE];
      s0 = fmaf(x0, w0, s0), s1 = fmaf(x1, w1, s1), s2 = fmaf(x2, w2, s2), s3 = fmaf(x3, w3, s3);
    }
    for (; c < hidden; c += ME_WAVE) s0 = fmaf(to_float(row[c]), w[c], s0);
    const float s = wave_sum((s0 + s1) + (s2 + s3));
    if (lane == 0) z[e] = s;
  }
  __syncthreads();
  if (wave != 0) return;
  if (shared_gate && lane == 0) shared_gate[t] = 1.f / (1.f + expf(-z[E]));
  if (scoring == RF_SCORE_SOFTMAX_ALL) {
    float zm = -INFINITY;
    for (int e = lane; e < E; e += ME_WAVE) zm = fmaxf(zm, z[e]);
    zm = wave_max(zm);
    float zs = 0.f;
    for (int e = lane; e < E; e += ME_WAVE) {
      sc[e] = expf(z[e] - zm);
      zs += sc[e];
    }
    zs = wave_sum(zs);
    for (int e = lane; e < E; e += ME_WAVE) {
      sc[e] = sc[e] / zs;
      z[e] = sc[e] + (correction ? correction[e] : 0.f);  // what the picks go by
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
  if (scoring == RF_SCORE_SIGMOID) {
    // scores sigmoid(z); the experts form n_groups equal groups of neighbours, a group's score is the sum of its two largest
    // scores, and only experts of the keep_groups best groups can be picked (the lower index among equals, as for the picks)
    for (int e = lane; e < E; e += ME_WAVE) sc[e] = 1.f / (1.f + expf(-z[e]));
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);
    if (n_groups > 1 && keep_groups < n_groups) {
      const int per = E / n_groups;
      for (int g = lane; g < n_groups; g += ME_WAVE) {
        float a = -INFINITY, b = -INFINITY;  // the largest and the second largest
        for (int i = 0; i < per; ++i) {
          const float v = sc[g * per + i];
          if (v > a) b = a, a = v;
          else if (v > b) b = v;
        }
        gs[g] = per > 1 ? a + b : a;
      }
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_s_waitcnt(0xc07f);
      for (int j = 0; j < keep_groups; ++j) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int g = lane; g < n_groups; g += ME_WAVE)
          if (gs[g] > best) best = gs[g], at = g;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
          const float ob = __shfl_xor(best, off, ME_WAVE);
          const int oa = __shfl_xor(at, off, ME_WAVE);
          if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
        }
        if (at >= n_groups) break;  // (a row of NaNs)
        if (lane == 0) gs[at] = -INFINITY;  // taken: its experts stay
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);
      }
      for (int e = lane; e < E; e += ME_WAVE)
        if (gs[e / per] != -INFINITY) z[e] = -INFINITY;  // a group that was not taken
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_s_waitcnt(0xc07f);
    }
  }
  float mine = 0.f, zmax = 0.f, sum = 0.f;  // lane j keeps the weight of the j-th pick
  int mine_e = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += ME_WAVE)
      if (z[e] > best) best = z[e], at = e;  // (ascending e: the lowest index among a lane's equals)
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, ME_WAVE);
      const int oa = __shfl_xor(at, off, ME_WAVE);
      if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
    }
    if (at >= E) at = 0;  // (a row of NaNs, as rows that pad a replayed step may be: any expert)
    if (j == 0) zmax = best;
    // the pick's weight before it is divided by the picks' sum: exp(z - z_max), or the pick's score
    const float p = scoring != RF_SCORE_SOFTMAX ? sc[at] : expf(best - zmax);
    if (lane == j) mine = p, mine_e = at;
    sum += p;
    if (lane == 0) {
      ids[(size_t)t * top + j] = at;
      z[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
  if (lane < top)
    wts[(size_t)t * top + lane] = scoring == RF_SCORE_SIGMOID ? mine / (sum + 1e-20f) * route_scale
                                  : scoring == RF_SCORE_SOFTMAX_ALL ? mine * route_scale : mine / sum;
  // A step of very few pairs needs no sorting: every pair is a tile of its own, in the order of the pairs (plan and
  // sorted as routed_sort_kernel leaves them for tiles of one row).
  if (plan && lane < top) {
    const int pair = t * top + lane;
    plan[1 + 3 * pair] = mine_e < E_real ? mine_e : 0;  // (never an index beyond the experts that have tensors)
    plan[2 + 3 * pair] = pair;
    plan[3 + 3 * pair] = mine_e < E_real ? 1 : 0;  // (an identity expert: a tile of no rows)
    sorted[pair] = pair;
    if (pair == 0) plan[0] = num_pairs;
  }
}

// plan: [0] number of tiles; [1 + 3 i ..] tile i: expert, first position, pairs; sorted [P]: the pair at each position.
__global__ __launch_bounds__(1024) void routed_sort_kernel(const int* __restrict__ ids, int P, int E_real, int max_tiles, int tile_rows,
                                                           int* __restrict__ plan, int* __restrict__ sorted, int n_identity = 0) {
  __shared__ int count[RF_MAX_EXPERTS], first[RF_MAX_EXPERTS];
  const int E = E_real + n_identity;  // (pairs of identity experts are counted and placed, but get no tiles)
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&count[ids[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      first[e] = at;
      for (int b = 0; e < E_real && b < count[e] && tiles < max_tiles; b += tile_rows, ++tiles) {
        plan[1 + 3 * tiles] = e;
        plan[2 + 3 * tiles] = at + b;
        plan[3 + 3 * tiles] = min(tile_rows, count[e] - b);
      }
      at += count[e];
    }
    plan[0] = tiles;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = first[e];
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) sorted[atomicAdd(&count[ids[p]], 1)] = p;
}

// Grid (tiles, tiles of 64 columns of ff). W_gu [E, 2 ff, hidden]: an expert's gate rows, then its up rows.
template <typename T>
__global__ __launch_bounds__(256) void routed_gate_up_kernel(const T* __restrict__ h, const T* __restrict__ W_gu,
                                                             const int* __restrict__ plan, const int* __restrict__ sorted,
                                                             T* __restrict__ acts, int hidden, int ff, int top, int act, float limit) {
  __shared__ TileLds lds;
  const int tile = blockIdx.x;
  if (tile >= plan[0]) return;
  const int e = plan[1 + 3 * tile], begin = plan[2 + 3 * tile], rows = plan[3 + 3 * tile];
  if (rows <= 0) return;  // (the pair of an identity expert, where the router wrote the list itself: no weights to read)
  const int c0 = blockIdx.y * TP_COLS, cols = min(TP_COLS, ff - c0);
  auto row_ptr = [&](int i) { return h + (size_t)(sorted[begin + i] / top) * hidden; };
  const bool ungated = act_is_ungated(act);  // W_gu is [E, ff, hidden] then: up rows alone
  const T* Wg = W_gu + ((size_t)e * (ungated ? 1 : 2) * ff + c0) * hidden;
  float g[4], u[4] = {0.f, 0.f, 0.f, 0.f};
  tile_product<T>(row_ptr, rows, Wg, cols, hidden, g, lds);
  if (!ungated) tile_product<T>(row_ptr, rows, Wg + (size_t)ff * hidden, cols, hidden, u, lds);
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  if (tx >= cols) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = ty + 4 * i;
    if (row < rows)
      acts[(size_t)(begin + row) * ff + c0 + tx] = from_float<T>(ungated ? ungated_act(g[i], act) : gated_pair(g[i], u[i], act, limit));
  }
}

// Grid (tiles, tiles of 64 columns of hidden). W_down [E, hidden, ff]. parts float32 [top, tokens, hidden].
template <typename T>
__global__ __launch_bounds__(256) void routed_down_kernel(const T* __restrict__ acts, const T* __restrict__ W_down,
                                                          const int* __restrict__ plan, const int* __restrict__ sorted,
                                                          const float* __restrict__ wts, float* __restrict__ parts, int num_tokens,
                                                          int hidden, int ff, int top) {
  __shared__ TileLds lds;
  const int tile = blockIdx.x;
  if (tile >= plan[0]) return;
  const int e = plan[1 + 3 * tile], begin = plan[2 + 3 * tile], rows = plan[3 + 3 * tile];
  if (rows <= 0) return;  // (the pair of an identity expert, where the router wrote the list itself: no weights to read)
  const int c0 = blockIdx.y * TP_COLS, cols = min(TP_COLS, hidden - c0);
  float acc[4];
  tile_product<T>([&](int i) { return acts + (size_t)(begin + i) * ff; }, rows, W_down + ((size_t)e * hidden + c0) * ff, cols, ff,
                  acc, lds);
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  if (tx >= cols) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = ty + 4 * i;
    if (row < rows) {
      const int pair = sorted[begin + row];
      parts[((size_t)(pair % top) * num_tokens + pair / top) * hidden + c0 + tx] = wts[pair] * acc[i];
    }
  }
}

// The two products on the matrix cores (bfloat16; hidden and ff multiples of 8): a tile is up to 16 * MT pairs of one expert,
// a block takes 64 columns of it, a wave 16 (tile_product.h: wave_product_bf16). GATED: rows of h gathered by the pairs'
// tokens, gate and up rows of the same columns side by side, act(gate) * up -> acts; else rows of acts, the down rows,
// weight * product -> parts. Tiles of 64 pairs (prompts) read an expert's weights a quarter as often as tiles of 16.
// MODE 0: the down product; 1: gate and up rows; 2: up rows alone (an expert without a gate: act(up) -> acts).
template <int MT, int MODE>
__global__ __launch_bounds__(256) void routed_tile_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                                                               const int* __restrict__ plan, const int* __restrict__ sorted,
                                                               const float* __restrict__ wts, bf16_t* __restrict__ acts,
                                                               float* __restrict__ parts, int num_tokens, int N, int K, int top,
                                                               int act, float limit) {
  const int tile = blockIdx.x;
  if (tile >= plan[0]) return;
  const int e = plan[1 + 3 * tile], begin = plan[2 + 3 * tile], rows = plan[3 + 3 * tile];
  if (rows <= 0) return;  // (the pair of an identity expert, where the router wrote the list itself: no weights to read)
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1), r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.y * 64 + wave * 16;
  if (n0 >= N) return;
  constexpr bool GATED = MODE == 1, GATHER = MODE != 0;
  constexpr int ACCS = GATED ? 2 : 1;
  const bf16_t* wrow[ACCS];
  const bf16_t* w0 = n0 + r < N ? W + ((size_t)e * ACCS * N + n0 + r) * K : nullptr;
  wrow[0] = w0;
  if (GATED) wrow[ACCS - 1] = w0 ? w0 + (size_t)N * K : nullptr;
  const bf16_t* xrow[MT];
  int pair[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = t * 16 + r;
    pair[t] = row < rows ? sorted[begin + row] : -1;
    xrow[t] = row < rows ? x + (GATHER ? (size_t)(pair[t] / top) : (size_t)(begin + row)) * K : nullptr;
  }
  tp_float4 acc[MT][ACCS];
  wave_product_bf16<MT, ACCS>(xrow, wrow, K, acc);
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    if (pair[t] < 0) continue;
    const int row = t * 16 + r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = n0 + 4 * g + i;
      if (col >= N) continue;
      if (GATED)
        acts[(size_t)(begin + row) * N + col] = from_float<bf16_t>(gated_pair(acc[t][0][i], acc[t][ACCS - 1][i], act, limit));
      else if (GATHER)
        acts[(size_t)(begin + row) * N + col] = from_float<bf16_t>(ungated_act(acc[t][0][i], act));
      else
        parts[((size_t)(pair[t] % top) * num_tokens + pair[t] / top) * N + col] = wts[pair[t]] * acc[t][0][i];
    }
  }
}

// Tiles of up to 16 pairs (decode steps): a block takes 16 columns of a tile and its four waves cut k among them in
// interleaved chunks of 32 (a wave alone walks a row of weights in k / 64 dependent trips to memory; four waves in a
// quarter of them), then add their sums up through LDS in the order of the waves. Otherwise as the kernel above.
template <int MODE>
__global__ __launch_bounds__(256) void routed_tile_ksplit_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                                                                 const int* __restrict__ plan, const int* __restrict__ sorted,
                                                                 const float* __restrict__ wts, bf16_t* __restrict__ acts,
                                                                 float* __restrict__ parts, int num_tokens, int N, int K, int top,
                                                                 int act, float limit) {
  constexpr bool GATED = MODE == 1, GATHER = MODE != 0;
  constexpr int ACCS = GATED ? 2 : 1, WAVES = 4, U = 2;
  __shared__ float red[WAVES][ACCS][64][4];
  const int tile = blockIdx.x;
  if (tile >= plan[0]) return;
  const int e = plan[1 + 3 * tile], begin = plan[2 + 3 * tile], rows = plan[3 + 3 * tile];
  if (rows <= 0) return;  // (the pair of an identity expert, where the router wrote the list itself: no weights to read)
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1), r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.y * 16;
  const bf16_t* w0 = n0 + r < N ? W + ((size_t)e * ACCS * N + n0 + r) * K : nullptr;
  const bf16_t* w1 = GATED && w0 ? w0 + (size_t)N * K : nullptr;
  const int pair = r < rows ? sorted[begin + r] : -1;
  const bf16_t* xr = r < rows ? x + (GATHER ? (size_t)(pair / top) : (size_t)(begin + r)) * K : nullptr;
  tp_float4 acc[ACCS];
#pragma unroll
  for (int a = 0; a < ACCS; ++a) acc[a] = (tp_float4){0.f, 0.f, 0.f, 0.f};
  const int chunks = (K + 31) / 32;
  for (int c0 = wave; c0 < chunks; c0 += WAVES * U) {
    tp_bf16x8 wf[U][ACCS], xf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + WAVES * u, at = c * 32 + 8 * g;
      const bool k_ok = c < chunks && at < K;
      wf[u][0] = tp_bf16x8{};
      if (w0 && k_ok) wf[u][0] = *reinterpret_cast<const tp_bf16x8*>(w0 + at);
      if (GATED) {
        wf[u][ACCS - 1] = tp_bf16x8{};
        if (w1 && k_ok) wf[u][ACCS - 1] = *reinterpret_cast<const tp_bf16x8*>(w1 + at);
      }
      xf[u] = tp_bf16x8{};
      if (xr && k_ok) xf[u] = *reinterpret_cast<const tp_bf16x8*>(xr + at);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int a = 0; a < ACCS; ++a) acc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][a], xf[u], acc[a], 0, 0, 0);
  }
#pragma unroll
  for (int a = 0; a < ACCS; ++a)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][a][lane][i] = acc[a][i];
  __syncthreads();
  if (wave != 0 || pair < 0) return;
  float sum[ACCS][4];
#pragma unroll
  for (int a = 0; a < ACCS; ++a)
#pragma unroll
    for (int i = 0; i < 4; ++i) sum[a][i] = ((red[0][a][lane][i] + red[1][a][lane][i]) + red[2][a][lane][i]) + red[3][a][lane][i];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int col = n0 + 4 * g + i;
    if (col >= N) continue;
    if (GATED)
      acts[(size_t)(begin + r) * N + col] = from_float<bf16_t>(gated_pair(sum[0][i], sum[ACCS - 1][i], act, limit));
    else if (GATHER)
      acts[(size_t)(begin + r) * N + col] = from_float<bf16_t>(ungated_act(sum[0][i], act));
    else
      parts[((size_t)(pair % top) * num_tokens + pair / top) * N + col] = wts[pair] * sum[0][i];
  }
}

extern "C" int me_routed_ff_max_tiles(long long tokens, int E, int top) {
  return (int)((tokens * top + TP_ROWS - 1) / TP_ROWS) + E + RF_DIRECT_PAIRS;  // (or a tile a pair, for steps of very few pairs)
}

// Bytes of workspace: ids and weights of the pairs, the tile list, the sorted pairs, the activations.
extern "C" long long me_routed_ff_workspace(long long tokens, int E, int top, int ff, int elem) {
  const long long P = tokens * top;
  const long long ints = P + P + 1 + 3ll * me_routed_ff_max_tiles(tokens, E, top) + P;
  return ints * 4 + 256 + P * ff * elem + 256;
}

// h [T, hidden] -> parts float32 [top, T, hidden]. Wr float32 [E, hidden]; W_gu [E, 2 ff, hidden]; W_down [E, hidden, ff].
// limit: what an activation with a limit clamps by. scoring (RF_SCORE_*), n_groups, keep_groups, route_scale: how the picks are
// bounded and weighted. shared_gate (float32 [T] or null): Wr has one more row behind the experts', and the sigmoid of a
// token's product with it is written there (the gate of an expert that every token uses).
// The pairs of identity experts: parts [pick, token, :] = weight * h [token, :].
template <typename T>
__global__ __launch_bounds__(256) void routed_identity_kernel(const T* __restrict__ h, const int* __restrict__ ids, const float* __restrict__ wts,
                                                              float* __restrict__ parts, int num_tokens, int hidden, int E_real, int top) {
  const int pair = blockIdx.x;
  if (ids[pair] < E_real) return;
  const int t = pair / top;
  const float w = wts[pair];
  float* dst = parts + ((size_t)(pair % top) * num_tokens + t) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = w * to_float(h[(size_t)t * hidden + i]);
}

// As me_routed_ff_scored. With scoring RF_SCORE_SOFTMAX_ALL the router (Wr float32 [E + n_identity, hidden]) has n_identity more outputs
// behind the experts', which stand for identity experts, and `correction` (float32 [E + n_identity] or null) is added to the scores
// for the choice alone. An activation code of MeAct (no gate): W_gu is [E, ff, hidden], the experts' up rows alone.
extern "C" int me_routed_ff_routed(const void* h, const float* Wr, const void* W_gu, const void* W_down, float* parts, void* workspace,
                                   int num_tokens, int hidden, int E, int top, int ff, int act, float limit, int scoring, int n_groups,
                                   int keep_groups, float route_scale, float* shared_gate, int n_identity, const float* correction,
                                   int dtype, hipStream_t stream);

extern "C" int me_routed_ff_scored(const void* h, const float* Wr, const void* W_gu, const void* W_down, float* parts, void* workspace,
                                   int num_tokens, int hidden, int E, int top, int ff, int act, float limit, int scoring, int n_groups,
                                   int keep_groups, float route_scale, float* shared_gate, int dtype, hipStream_t stream) {
  return me_routed_ff_routed(h, Wr, W_gu, W_down, parts, workspace, num_tokens, hidden, E, top, ff, act, limit, scoring, n_groups, keep_groups,
                             route_scale, shared_gate, 0, nullptr, dtype, stream);
}

extern "C" int me_routed_ff_routed(const void* h, const float* Wr, const void* W_gu, const void* W_down, float* parts, void* workspace,
                                   int num_tokens, int hidden, int E, int top, int ff, int act, float limit, int scoring, int n_groups,
                                   int keep_groups, float route_scale, float* shared_gate, int n_identity, const float* correction,
                                   int dtype, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (scoring != RF_SCORE_SOFTMAX && scoring != RF_SCORE_SIGMOID && scoring != RF_SCORE_SOFTMAX_ALL) return me_fail("me_routed_ff: scoring %d", scoring);
  if (n_identity < 0 || (n_identity > 0 && scoring != RF_SCORE_SOFTMAX_ALL) || E + n_identity > RF_MAX_EXPERTS)
    return me_fail("me_routed_ff: %d identity experts beside %d experts", n_identity, E);
  const bool ungated = act_is_ungated(act);
  auto finish = [&]() {
    if (n_identity > 0) {  // (behind the router, beside the experts' products: rows that no tile writes)
      const long long pairs = (long long)num_tokens * top;
      if (dtype == ME_F32)
        routed_identity_kernel<float><<<(unsigned)pairs, 256, 0, stream>>>((const float*)h, (const int*)workspace, (const float*)((const int*)workspace + pairs),
                                                                           parts, num_tokens, hidden, E, top);
      else
        routed_identity_kernel<bf16_t><<<(unsigned)pairs, 256, 0, stream>>>((const bf16_t*)h, (const int*)workspace, (const float*)((const int*)workspace + pairs),
                                                                            parts, num_tokens, hidden, E, top);
    }
    return me_check_launch("me_routed_ff");
  };   if (scoring == RF_SCORE_SIGMOID && (n_groups < 1 || E % n_groups || keep_groups < 1 || keep_groups > n_groups ||
                                      (long long)keep_groups * (E / n_groups) < top))
    return me_fail("me_routed_ff: %d experts in %d groups of which %d are kept, %d picks", E, n_groups, keep_groups, top);
  if (E < 1 || E > RF_MAX_EXPERTS || top < 1 || top > RF_MAX_TOP || top > E + n_identity)
    return me_fail("me_routed_ff: %d experts (at most %d), %d of them a token (at most %d)", E, RF_MAX_EXPERTS, top, RF_MAX_TOP);
  if (hidden <= 0 || ff <= 0) return me_fail("me_routed_ff: hidden=%d ff=%d", hidden, ff);
  const long long P = (long long)num_tokens * top;
  const int max_tiles = me_routed_ff_max_tiles(num_tokens, E, top);
  int* ids = (int*)workspace;
  float* wts = (float*)(ids + P);
  int* plan = (int*)(wts + P);
  int* sorted = plan + 1 + 3 * (size_t)max_tiles;
  const size_t elem = dtype == ME_F32 ? 4 : 2;
  char* acts = (char*)(((uintptr_t)(sorted + P) + 255) & ~(uintptr_t)255);
  const dim3 g_up(max_tiles, (ff + TP_COLS - 1) / TP_COLS), g_down(max_tiles, (hidden + TP_COLS - 1) / TP_COLS);
  if (g_up.y > 65535 || g_down.y > 65535) return me_fail("me_routed_ff: hidden=%d ff=%d", hidden, ff);
  (void)elem;
  // few tokens (decode steps): a wave an expert, so that all of a token's logits are on their way at once
  const int route_threads = num_tokens <= 64 ? 64 * (E < 16 ? (E < 4 ? 4 : E) : 16) : 256;
  const bool aligned = ((((uintptr_t)h | (uintptr_t)W_gu | (uintptr_t)W_down | (uintptr_t)acts) & 15) == 0);
  if (dtype == ME_BF16 && hidden % 8 == 0 && ff % 8 == 0 && aligned) {  // the matrix cores
    const int wide = P >= 32ll * E;  // 32 and more pairs an expert on average: tiles of 64 pairs
    const bool direct = P <= RF_DIRECT_PAIRS && (ff + 15) / 16 <= 65535 && (hidden + 15) / 16 <= 65535;
    routed_route_kernel<bf16_t><<<num_tokens, route_threads, 0, stream>>>((const bf16_t*)h, Wr, ids, wts, hidden, E, top,
                                                                            direct ? plan : nullptr, direct ? sorted : nullptr, (int)P,
                                                                            scoring, n_groups, keep_groups, route_scale, shared_gate, n_identity, correction);
    if (direct) {  // the router has written the list of tiles itself
      const dim3 k_up((unsigned)P, (ff + 15) / 16), k_down((unsigned)P, (hidden + 15) / 16);
      if (ungated) routed_tile_ksplit_kernel<2><<<k_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts, nullptr, num_tokens, ff, hidden, top, act, limit);
      else routed_tile_ksplit_kernel<1><<<k_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts,
                                                                nullptr, num_tokens, ff, hidden, top, act, limit);
      routed_tile_ksplit_kernel<0><<<k_down, 256, 0, stream>>>((const bf16_t*)acts, (const bf16_t*)W_down, plan, sorted, wts, nullptr,
                                                                 parts, num_tokens, hidden, ff, top, act, limit);
      return finish();
    }
    if (P >= 96ll * E && hidden % 64 == 0 && ff % 64 == 0) {
      // prompts: tiles of 128 pairs through the product that stages both operands in LDS (gemm_grouped.hip)
      const int rows128 = me_gemm_grouped_tile_rows(), tiles128 = (int)((P + rows128 - 1) / rows128) + E;
      routed_sort_kernel<<<1, 1024, 0, stream>>>(ids, (int)P, E, max_tiles, rows128, plan, sorted, n_identity);
      if (me_gemm_grouped_bf16(h, W_gu, plan, sorted, wts, acts, nullptr, num_tokens, ff, hidden, top, tiles128, act, limit, stream)) return 1;
      if (me_gemm_grouped_bf16(acts, W_down, plan, sorted, wts, nullptr, parts, num_tokens, hidden, ff, top, tiles128, 0, 0.f, stream)) return 1;
      return finish();
    }
    routed_sort_kernel<<<1, 1024, 0, stream>>>(ids, (int)P, E, max_tiles, wide ? 64 : 16, plan, sorted, n_identity);
    if (wide) {
      const unsigned tiles64 = (unsigned)((P + 63) / 64) + E;  // fewer tiles than the list's bound: whole blocks that only return
      const dim3 g_up(tiles64, (ff + TP_COLS - 1) / TP_COLS), g_down(tiles64, (hidden + TP_COLS - 1) / TP_COLS);
      if (ungated) routed_tile_mfma_kernel<4, 2><<<g_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts, nullptr, num_tokens, ff, hidden, top, act, limit);
      else routed_tile_mfma_kernel<4, 1><<<g_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts,
                                                                 nullptr, num_tokens, ff, hidden, top, act, limit);
      routed_tile_mfma_kernel<4, 0><<<g_down, 256, 0, stream>>>((const bf16_t*)acts, (const bf16_t*)W_down, plan, sorted, wts, nullptr,
                                                                  parts, num_tokens, hidden, ff, top, act, limit);
    } else if (P <= 4ll * E && (ff + 15) / 16 <= 65535 && (hidden + 15) / 16 <= 65535) {
      // few pairs (decode steps): most tiles hold a pair or two, and what a step waits for is the walk over k
      const dim3 k_up(max_tiles, (ff + 15) / 16), k_down(max_tiles, (hidden + 15) / 16);
      if (ungated) routed_tile_ksplit_kernel<2><<<k_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts, nullptr, num_tokens, ff, hidden, top, act, limit);
      else routed_tile_ksplit_kernel<1><<<k_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts,
                                                                nullptr, num_tokens, ff, hidden, top, act, limit);
      routed_tile_ksplit_kernel<0><<<k_down, 256, 0, stream>>>((const bf16_t*)acts, (const bf16_t*)W_down, plan, sorted, wts, nullptr,
                                                                 parts, num_tokens, hidden, ff, top, act, limit);
    } else {
      if (ungated) routed_tile_mfma_kernel<1, 2><<<g_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts, nullptr, num_tokens, ff, hidden, top, act, limit);
      else routed_tile_mfma_kernel<1, 1><<<g_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, wts, (bf16_t*)acts,
                                                                 nullptr, num_tokens, ff, hidden, top, act, limit);
      routed_tile_mfma_kernel<1, 0><<<g_down, 256, 0, stream>>>((const bf16_t*)acts, (const bf16_t*)W_down, plan, sorted, wts, nullptr,
                                                                  parts, num_tokens, hidden, ff, top, act, limit);
    }
    return finish();
  }
  if (dtype == ME_F32) {
    routed_route_kernel<float><<<num_tokens, route_threads, 0, stream>>>((const float*)h, Wr, ids, wts, hidden, E, top, nullptr, nullptr, 0,
                                                                         scoring, n_groups, keep_groups, route_scale, shared_gate, n_identity, correction);
    routed_sort_kernel<<<1, 1024, 0, stream>>>(ids, (int)P, E, max_tiles, TP_ROWS, plan, sorted, n_identity);
    routed_gate_up_kernel<float><<<g_up, 256, 0, stream>>>((const float*)h, (const float*)W_gu, plan, sorted, (float*)acts, hidden, ff,
                                                            top, act, limit);
    routed_down_kernel<float><<<g_down, 256, 0, stream>>>((const float*)acts, (const float*)W_down, plan, sorted, wts, parts,
                                                          num_tokens, hidden, ff, top);
  } else {
    routed_route_kernel<bf16_t><<<num_tokens, route_threads, 0, stream>>>((const bf16_t*)h, Wr, ids, wts, hidden, E, top, nullptr, nullptr, 0,
                                                                          scoring, n_groups, keep_groups, route_scale, shared_gate, n_identity, correction);
    routed_sort_kernel<<<1, 1024, 0, stream>>>(ids, (int)P, E, max_tiles, TP_ROWS, plan, sorted, n_identity);
    routed_gate_up_kernel<bf16_t><<<g_up, 256, 0, stream>>>((const bf16_t*)h, (const bf16_t*)W_gu, plan, sorted, (bf16_t*)acts, hidden,
                                                             ff, top, act, limit);
    routed_down_kernel<bf16_t><<<g_down, 256, 0, stream>>>((const bf16_t*)acts, (const bf16_t*)W_down, plan, sorted, wts, parts,
                                                           num_tokens, hidden, ff, top);
  }
  return finish();
}

extern "C" int me_routed_ff(const void* h, const float* Wr, const void* W_gu, const void* W_down, float* parts, void* workspace,
                            int num_tokens, int hidden, int E, int top, int ff, int act, int dtype, hipStream_t stream) {
  return me_routed_ff_scored(h, Wr, W_gu, W_down, parts, workspace, num_tokens, hidden, E, top, ff, act, 0.f, RF_SCORE_SOFTMAX, 1, 1,
                             1.f, nullptr, dtype, stream);
}

// An expert that every token uses, behind its ungated product: gu [T, 2 ff] (gate columns, then up columns) ->
// act [T, ff] = gated_pair(gate, up) * row_gate[t] (row_gate float32 [T] or null: 1).
template <typename T>
__global__ __launch_bounds__(256) void gated_rows_kernel(const T* __restrict__ gu, const float* __restrict__ row_gate,
                                                         T* __restrict__ act_out, long long total, int ff, int act, float limit) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long long t = i / ff;
  const int c = (int)(i % ff);
  const float g = to_float(gu[t * 2 * ff + c]), u = to_float(gu[t * 2 * ff + ff + c]);
  const float y = gated_pair(g, u, act, limit) * (row_gate ? row_gate[t] : 1.f);
  act_out[i] = from_float<T>(y);
}

extern "C" int me_gated_rows(const void* gu, const float* row_gate, void* act_out, int num_tokens, int ff, int act, float limit, int dtype,
                             hipStream_t stream) {
  if (num_tokens <= 0 || ff <= 0) return 0;
  const long long total = (long long)num_tokens * ff;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == ME_F32)
    gated_rows_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, row_gate, (float*)act_out, total, ff, act, limit);
  else
    gated_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, row_gate, (bf16_t*)act_out, total, ff, act, limit);
  return me_check_launch("me_gated_rows");
}
