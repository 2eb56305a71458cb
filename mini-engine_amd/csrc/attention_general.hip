// Causal grouped-query attention over the paged cache, for any mix of items in a step: one wave, or a
// block of eight, per (new token, query head). It takes every size the cache allows (any page size, any group
// size, head sizes up to 256 in steps of 2) in float32 or bfloat16 storage, and is the kernel of
// the 32-bit path; the bfloat16 path uses the matrix-core kernels where their size limits hold.
//
// A token at absolute position p of item b sees keys lo..p of item b, lo = max(0, p - window + 1)
// (window == 0: lo = 0). Keys are visited in tiles of 64 aligned to absolute position (tile t holds
// positions 64t .. 64t+63), four tiles to a chunk (chunk c holds positions 256c .. 256c+255): the tiles of a
// chunk update a running (maximum, sum, weighted values) from nothing, and the chunks' results are merged in
// ascending order. So the order of every sum depends on p, lo and the head alone, never on how the sequence
// was cut into steps, on what else is in the batch, or on how many waves share the chunks of a token.
//
// Cache layout per layer: keys K[page, kv_head, slot, d]; values transposed V[page, kv_head, dv, slot] (dv: the
// value heads' size, which need not be the keys').
//
// Kept first tokens: with keep_first = f > 0 the keys 0 .. f-1 stay visible behind the window. Where the window still
// reaches them the visible keys are one run from 0; else they are two runs, 0 .. f-1 and lo .. p, and the chunks of the
// first run (aligned to absolute position like the others) come before those of the second.
//
// Values that were turned by their own position before they were cached (pairs of elements, by the angles of a table
// [positions, 2, dv/2]): the output of a token at position p, a sum of such values, is turned back by p's angles.
#include "common.h"

#define AG_MAX_D 256   // the kernels' usual instance: heads of up to 256 elements
#define AG_MAX_D_WIDE 512  // a second instance of the kernel with a wave per token and head: up to 512

#define AG_CHUNK 256  // keys per chunk

// One chunk's result into the running one, the same operations wherever it is called. With nothing before
// (mt = -inf, lt = 0, acct = 0) the chunk's result comes through unchanged: exp(-inf) = 0 and exp(0) = 1.
template <int KMAX>
__device__ __forceinline__ void ag_merge(float& mt, float& lt, float (&acct)[KMAX], float mc, float lc,
                                         const float (&accc)[KMAX]) {
  const float mn = fmaxf(mt, mc);
  const float at = expf(mt - mn), ac = expf(mc - mn);
  lt = fmaf(lt, at, lc * ac);
#pragma unroll
  for (int k = 0; k < KMAX; ++k) acct[k] = fmaf(acct[k], at, accc[k] * ac);
  mt = mn;
}

// `wpu` waves per (token, head): 1 (a block of four waves serves four of them), or all waves of the block for one,
// which then take the chunks in turns, a round of wpu chunks at a time, and wave 0 merges the round's results in order.
template <typename T, int KMAX>
__global__ __launch_bounds__(512) void attention_general_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table,
    int table_width, T* __restrict__ out, int num_tokens, int nh, int nkv, int d, int dv, int bs, int window, int keep_first,
    const float* __restrict__ unturn, int un_pairing, float scale, int wpu, const float* __restrict__ sink,
    const T* __restrict__ gate, size_t gate_row, const T* __restrict__ k_pool, const T* __restrict__ v_pool, int pool,
    long long out_row, int out_col, float out_scale, float softcap) {
  constexpr int DMAX = KMAX * ME_WAVE;  // the largest head this instance takes
  __shared__ float qs[8][DMAX];
  __shared__ float parts[8][DMAX + 2];  // with several waves per unit: a round's results (values, maximum, sum)
  const int wave = threadIdx.x / ME_WAVE, lane = threadIdx.x & (ME_WAVE - 1);
  const int w = wave % wpu;
  const long long unit = (long long)blockIdx.x * (blockDim.x / ME_WAVE / wpu) + wave / wpu;
  if (unit >= (long long)num_tokens * nh) return;  // (with several waves per unit: the whole block)
  const int t = (int)(unit / nh), head = (int)(unit % nh);
  const int kvh = head / (nh / nkv);
  const int p = positions[t];
  int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  int kept = keep_first < lo ? keep_first : lo;  // keys 0 .. kept-1 are visible beside lo .. p
  if (kept == lo) lo = 0, kept = 0;              // the two runs meet: one run from 0
  // Pooled blocks: entry b of the pooled pages stands for the positions b pool .. b pool + pool - 1 and is visible once the
  // window has passed all of them. The entries 0 .. kept-1 are a run of their own, walked like kept first keys.
  if (pool > 0) kept = lo / pool;
  const int kept_chunks = (kept + AG_CHUNK - 1) / AG_CHUNK;
  const int* table = block_table + (size_t)token_item[t] * table_width;

  const T* qrow = q + ((size_t)t * nh + head) * d;
  float* qw = qs[wave];
  for (int i = lane; i < d; i += ME_WAVE) qw[i] = to_float(qrow[i]) * scale;
  __builtin_amdgcn_wave_barrier();

  float mt = -INFINITY, lt = 0.f;
  float acct[KMAX];
#pragma unroll
  for (int k = 0; k < KMAX; ++k) acct[k] = 0.f;

  const bool vec_k = sizeof(T) == 4 && d % 4 == 0 && ((uintptr_t)k_cache & 15) == 0;   // a key row in 16-byte pieces
  const bool vec_v = sizeof(T) == 4 && bs % 4 == 0 && ((uintptr_t)v_cache & 15) == 0;  // four keys of a value row at once
  const int first_chunk = lo / AG_CHUNK, n_chunks = kept_chunks + p / AG_CHUNK - first_chunk + 1;
  for (int round = 0; round * wpu < n_chunks; ++round) {
    const int ci = round * wpu + w;  // this wave's chunk of the round, if there is one
    float m = -INFINITY, l = 0.f;
    float acc[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) acc[k] = 0.f;
    const bool of_kept = ci < kept_chunks;  // a chunk of the kept first keys, else of the run lo .. p
    const int chunk0 = (of_kept ? ci : first_chunk + ci - kept_chunks) * AG_CHUNK;
    const int vlo = of_kept ? 0 : lo, vhi = of_kept ? kept - 1 : p;  // the run's visible keys
    const int tile_first = ci < n_chunks ? max(chunk0, (vlo / 64) * 64) : 1;  // (no chunk left for this wave: no tiles)
    const int tile_last = ci < n_chunks ? min(vhi, chunk0 + AG_CHUNK - 1) : 0;
    for (int tile = tile_first; tile <= tile_last; tile += 64) {
      const int key = tile + lane;
      const bool valid = key >= vlo && key <= vhi;
      float s = -INFINITY;
      const T* kc = of_kept && pool > 0 ? k_pool : k_cache;
      const T* vc = of_kept && pool > 0 ? v_pool : v_cache;
      if (valid) {
        const int page = table[key / bs];
        const T* krow = kc + (((size_t)page * nkv + kvh) * bs + key % bs) * d;
        float dot = 0.f;
        if (vec_k) {  // the same products in the same order; 128 elements of the row are requested before the first is used
          const float4* k4 = reinterpret_cast<const float4*>(krow);
          const int n4 = d / 4;
          for (int base = 0; base < n4; base += 32) {
            float4 kv[32];
#pragma unroll
            for (int u = 0; u < 32; ++u) kv[u] = base + u < n4 ? k4[base + u] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int u = 0; u < 32; ++u)
              if (base + u < n4) {
                const int i = 4 * (base + u);
                dot = fmaf(qw[i], kv[u].x, dot);
                dot = fmaf(qw[i + 1], kv[u].y, dot);
                dot = fmaf(qw[i + 2], kv[u].z, dot);
                dot = fmaf(qw[i + 3], kv[u].w, dot);
              }
          }
        } else {
          for (int i = 0; i < d; ++i) dot = fmaf(qw[i], to_float(krow[i]), dot);
        }
        s = softcap > 0.f ? softcap * tanhf(dot / softcap) : dot;  // (bounded scores: the scaled score through a tanh)
      }
      const float m_new = fmaxf(m, wave_max(s));  // at least one key of the tile is visible
      const float pr = valid ? expf(s - m_new) : 0.f;
      const float alpha = expf(m - m_new);  // exp(-inf) = 0 on the first tile
      l = l * alpha + wave_sum(pr);
#pragma unroll
      for (int k = 0; k < KMAX; ++k) acc[k] *= alpha;
      m = m_new;
      const int j_lo = vlo > tile ? vlo - tile : 0;
      const int j_hi = vhi - tile < 63 ? vhi - tile : 63;
      int j = j_lo;
      if (vec_v) {
        // whole groups of four keys that lie in one page (tiles and groups are aligned to 4, pages hold a multiple of
        // 4): one 16-byte load per group and element of the head, the sums in the order of the keys as below
        for (; j <= j_hi && (j & 3); ++j) {
          const float pj = __shfl(pr, j, ME_WAVE);
          const int kj = tile + j;
          const T* vbase = vc + ((size_t)table[kj / bs] * nkv + kvh) * dv * bs + kj % bs;
#pragma unroll
          for (int k = 0; k < KMAX; ++k) {
            const int i = lane + k * ME_WAVE;
            if (i < dv) acc[k] = fmaf(pj, to_float(vbase[(size_t)i * bs]), acc[k]);
          }
        }
        // eight groups of four keys at a time: their values are requested before the first is used
        const int groups = j <= j_hi ? (j_hi + 1 - j) / 4 : 0;  // whole groups from j on
        for (int g0 = 0; g0 < groups; g0 += 8) {
          float4 vv[8][KMAX];
#pragma unroll
          for (int gq = 0; gq < 8; ++gq) {
            const bool there = g0 + gq < groups;
            const int kj = tile + j + 4 * (there ? g0 + gq : 0);
            const T* vbase = vc + ((size_t)table[kj / bs] * nkv + kvh) * dv * bs + kj % bs;
#pragma unroll
            for (int k = 0; k < KMAX; ++k) {
              const int i = lane + k * ME_WAVE;
              vv[gq][k] = make_float4(0.f, 0.f, 0.f, 0.f);
              if (there && i < dv) vv[gq][k] = *reinterpret_cast<const float4*>(vbase + (size_t)i * bs);
            }
          }
#pragma unroll
          for (int gq = 0; gq < 8; ++gq) {
            if (g0 + gq < groups) {
              const int jj = j + 4 * (g0 + gq);
              const float p0 = __shfl(pr, jj, ME_WAVE), p1 = __shfl(pr, jj + 1, ME_WAVE), p2 = __shfl(pr, jj + 2, ME_WAVE),
                          p3 = __shfl(pr, jj + 3, ME_WAVE);
#pragma unroll
              for (int k = 0; k < KMAX; ++k) {
                if (lane + k * ME_WAVE < dv) {
                  acc[k] = fmaf(p0, vv[gq][k].x, acc[k]);
                  acc[k] = fmaf(p1, vv[gq][k].y, acc[k]);
                  acc[k] = fmaf(p2, vv[gq][k].z, acc[k]);
                  acc[k] = fmaf(p3, vv[gq][k].w, acc[k]);
                }
              }
            }
          }
        }
        j += 4 * groups;
      }
      for (; j <= j_hi; ++j) {
        const float pj = __shfl(pr, j, ME_WAVE);
        const int kj = tile + j;
        const int page = table[kj / bs];
        const T* vbase = vc + ((size_t)page * nkv + kvh) * dv * bs + kj % bs;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          const int i = lane + k * ME_WAVE;
          if (i < dv) acc[k] = fmaf(pj, to_float(vbase[(size_t)i * bs]), acc[k]);
        }
      }
    }
    if (wpu == 1) {
      ag_merge<KMAX>(mt, lt, acct, m, l, acc);
    } else {  // the round's results go through LDS to wave 0, which merges them in the order of their chunks
      if (ci < n_chunks) {
#pragma unroll
        for (int k = 0; k < KMAX; ++k) parts[w][lane + k * ME_WAVE] = acc[k];
        if (lane == 0) parts[w][DMAX] = m, parts[w][DMAX + 1] = l;
      }
      __syncthreads();
      if (w == 0)
        for (int o = 0; o < wpu && round * wpu + o < n_chunks; ++o) {
          float accc[KMAX];
#pragma unroll
          for (int k = 0; k < KMAX; ++k) accc[k] = parts[o][lane + k * ME_WAVE];
          ag_merge<KMAX>(mt, lt, acct, parts[o][DMAX], parts[o][DMAX + 1], accc);
        }
      __syncthreads();
    }
  }
  if (w != 0) return;
  T* orow = out + (size_t)t * out_row + out_col + (size_t)head * dv;
  if (sink) {  // one more term exp(sink) in the denominator, with no value: a chunk of its own, merged last
    float none[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) none[k] = 0.f;
    ag_merge<KMAX>(mt, lt, acct, sink[head], 1.f, none);
  }
  float inv = out_scale / lt;
  if (gate) inv *= 1.f / (1.f + expf(-to_float(gate[(size_t)t * gate_row + head])));  // the head's output gate
  if (unturn) {  // the sum of turned values, turned back by this token's angles: through this wave's row of LDS
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int i = lane + k * ME_WAVE;
      if (i < dv) qw[i] = acct[k] * inv;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): LDS writes of this wave are visible
    const float* cs = unturn + (size_t)p * dv;  // [2, dv / 2] of this position
    const int half = dv / 2;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int i = lane + k * ME_WAVE;
      if (i < dv) {
        const bool first = un_pairing == 0 ? i < half : (i & 1) == 0;
        const int j = un_pairing == 0 ? (first ? i : i - half) : i >> 1;
        const int other = un_pairing == 0 ? (first ? i + half : i - half) : i ^ 1;
        const float c = cs[j], sn = cs[half + j];
        orow[i] = from_float<T>(first ? qw[i] * c + qw[other] * sn : qw[i] * c - qw[other] * sn);
      }
    }
    return;
  }
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int i = lane + k * ME_WAVE;
    if (i < dv) orow[i] = from_float<T>(acct[k] * inv);
  }
}

// The same attention for steps that bring several tokens per item (prompts, portions): a block takes up to
// `tq` consecutive tokens of the step and the heads of one kv head, a wave per (token, head), and stages each tile of
// 64 keys and values in LDS once for all of them, where the kernel above has every wave fetch its own copy (a 2,048-token
// prompt: 34 GB a layer from the L2). Tokens of a block that belong to different items are served one item after the
// other. Every wave does the arithmetic of the kernel above in the same order (the products of a score in ascending
// element, the keys of a tile in ascending position, the same reductions across lanes), so the two kernels give the same
// bits and a step may use either. float32, head sizes that are a multiple of 4, pages that hold a multiple of 4 keys.
constexpr int AS_KPAD = 4, AS_VROW = 68;  // LDS rows: a key's d + 4 floats, an element's 64 + 4 keys (16-byte reads of consecutive
                                           // rows by consecutive lanes without bank conflicts; 8 and 72 measured slower)

// DT: the head size if it is 64, 128 or 256 (loops unroll, no guards), else 0 (any multiple of 4 up to 256).
template <int DT>
__global__ __launch_bounds__(1024) void attention_shared_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k_cache, const float* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ token_item, const int* __restrict__ block_table,
    int table_width, float* __restrict__ out, int num_tokens, int nh, int nkv, int d_any, int bs, int bs_shift, int window,
    float scale, int tq) {
  constexpr int KMAX = DT ? DT / ME_WAVE : AG_MAX_D / ME_WAVE;  // elements of the output per lane
  const int d = DT ? DT : d_any, d4 = d / 4;
  extern __shared__ __attribute__((aligned(16))) float as_lds[];
  const int waves = blockDim.x / ME_WAVE;
  float* Ks = as_lds;                      // [64][d + AS_KPAD]
  float* Vs = Ks + 64 * (d + AS_KPAD);     // [d][AS_VROW]
  float* qs = Vs + (size_t)d * AS_VROW;    // [waves][d]
  float* ps = qs + (size_t)waves * d;      // [waves][64]: a tile's weights, for every lane to read
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / ME_WAVE), lane = threadIdx.x & (ME_WAVE - 1);
  const int group = nh / nkv, kvh = blockIdx.y;
  // (the step's last tokens first: they are the ones with the most keys before them, and blocks start in this order)
  const int first = (gridDim.x - 1 - blockIdx.x) * tq, limit = min(first + tq, num_tokens);
  const int t = first + wave / group, head = kvh * group + wave % group;
  const bool mine = wave < tq * group && t < limit;
  float* qw = qs + (size_t)wave * d;
  float* pw = ps + wave * 64;
  const int krow_floats = d + AS_KPAD;
  // staging: a wave copies whole key rows, 64 / dp rows at a time (dp: d4 rounded up to a power of two, lanes beyond d4 idle)
  int dp_shift = 0;
  while ((1 << dp_shift) < d4) ++dp_shift;
  const int k_rows_per_wave = ME_WAVE >> dp_shift, k_row_in_wave = lane >> dp_shift, k_piece = lane & ((1 << dp_shift) - 1);
  auto page_of = [&](int key, int& slot) {
    if (bs_shift >= 0) {
      slot = key & (bs - 1);
      return key >> bs_shift;
    }
    slot = key % bs;
    return key / bs;
  };

  for (int seg = first; seg < limit;) {  // runs of tokens of one item (every thread walks the same runs)
    const int item = token_item[seg];
    int seg_end = seg + 1;
    while (seg_end < limit && token_item[seg_end] == item) ++seg_end;
    const int* table = block_table + (size_t)item * table_width;
    int p_first = positions[seg], p_last = p_first;  // the run's lowest and highest position (a portion's are consecutive)
    for (int i = seg + 1; i < seg_end; ++i) p_first = min(p_first, positions[i]), p_last = max(p_last, positions[i]);
    const int lo_first = window > 0 ? max(p_first - window + 1, 0) : 0;
    const bool active = mine && t >= seg && t < seg_end;
    const int p = active ? __builtin_amdgcn_readfirstlane(positions[t]) : 0;
    const int lo = window > 0 ? max(p - window + 1, 0) : 0;
    if (active) {
      const float* qrow = q + ((size_t)t * nh + head) * d;
      for (int i = lane; i < d; i += ME_WAVE) qw[i] = qrow[i] * scale;
    }
    float m = -INFINITY, l = 0.f, mt = -INFINITY, lt = 0.f;  // the chunk in hand, and the chunks before it merged
    float acc[KMAX], acct[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) acc[k] = 0.f, acct[k] = 0.f;

    for (int tile = (lo_first / 64) * 64; tile <= p_last; tile += 64) {
      __syncthreads();  // every wave has left the tile before (and the q rows are written)
      for (int row = wave * k_rows_per_wave + k_row_in_wave; row < 64; row += waves * k_rows_per_wave) {
        const int key = tile + row;  // keys up to the last position of the run
        if (key <= p_last && k_piece < d4) {
          int slot;
          const int page = table[page_of(key, slot)];
          const float* src = k_cache + (((size_t)page * nkv + kvh) * bs + slot) * d + 4 * k_piece;
          *reinterpret_cast<float4*>(Ks + row * krow_floats + 4 * k_piece) = *reinterpret_cast<const float4*>(src);
        }
      }
      for (int idx = threadIdx.x; idx < d * 16; idx += blockDim.x) {  // four keys of an element at a time (they share a page)
        const int i = idx >> 4, key = tile + 4 * (idx & 15);
        if (key <= p_last) {
          int slot;
          const int page = table[page_of(key, slot)];
          const float* src = v_cache + ((size_t)page * nkv + kvh) * d * bs + (size_t)i * bs + slot;
          *reinterpret_cast<float4*>(Vs + i * AS_VROW + 4 * (idx & 15)) = *reinterpret_cast<const float4*>(src);
        }
      }
      __syncthreads();
      if (!active || tile > p || tile < (lo / 64) * 64) continue;
      if (tile % AG_CHUNK == 0 && tile > lo) {  // a chunk begins behind another one of this token: that one is complete
        ag_merge<KMAX>(mt, lt, acct, m, l, acc);
        m = -INFINITY, l = 0.f;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) acc[k] = 0.f;
      }
      const int key = tile + lane;
      const bool valid = key >= lo && key <= p;
      float s = -INFINITY;
      if (valid) {
        const float4* k4 = reinterpret_cast<const float4*>(Ks + lane * krow_floats);
        const float4* q4 = reinterpret_cast<const float4*>(qw);
        float dot = 0.f;
        for (int base = 0; base < d4; base += 8) {  // eight pieces of the row and of q are requested before the first is used
          float4 kv[8], qv[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int at = DT || base + u < d4 ? base + u : d4 - 1;
            kv[u] = k4[at], qv[u] = q4[at];
          }
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (DT || base + u < d4) {
              dot = fmaf(qv[u].x, kv[u].x, dot);
              dot = fmaf(qv[u].y, kv[u].y, dot);
              dot = fmaf(qv[u].z, kv[u].z, dot);
              dot = fmaf(qv[u].w, kv[u].w, dot);
            }
        }
        s = dot;
      }
      const float m_new = fmaxf(m, wave_max(s));
      const float pr = valid ? expf(s - m_new) : 0.f;
      const float alpha = expf(m - m_new);
      l = l * alpha + wave_sum(pr);
#pragma unroll
      for (int k = 0; k < KMAX; ++k) acc[k] *= alpha;
      m = m_new;
      pw[lane] = pr;
      __builtin_amdgcn_wave_barrier();
      const int j_lo = lo > tile ? lo - tile : 0;
      const int j_hi = p - tile < 63 ? p - tile : 63;
      int j = j_lo;
      for (; j <= j_hi && (j & 3); ++j) {
        const float pj = pw[j];
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          const int i = lane + k * ME_WAVE;
          if (DT || i < d) acc[k] = fmaf(pj, Vs[i * AS_VROW + j], acc[k]);
        }
      }
      for (; j + 15 <= j_hi; j += 16) {  // four groups of four keys: their values are requested before the first is used
        float4 vv[4][KMAX], pv[4];
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          pv[gq] = *reinterpret_cast<const float4*>(pw + j + 4 * gq);
#pragma unroll
          for (int k = 0; k < KMAX; ++k) {
            const int i = lane + k * ME_WAVE;
            vv[gq][k] = *reinterpret_cast<const float4*>(Vs + (DT || i < d ? i : 0) * AS_VROW + j + 4 * gq);
          }
        }
#pragma unroll
        for (int gq = 0; gq < 4; ++gq)
#pragma unroll
          for (int k = 0; k < KMAX; ++k)
            if (DT || lane + k * ME_WAVE < d) {
              acc[k] = fmaf(pv[gq].x, vv[gq][k].x, acc[k]);
              acc[k] = fmaf(pv[gq].y, vv[gq][k].y, acc[k]);
              acc[k] = fmaf(pv[gq].z, vv[gq][k].z, acc[k]);
              acc[k] = fmaf(pv[gq].w, vv[gq][k].w, acc[k]);
            }
      }
      for (; j + 3 <= j_hi; j += 4) {
        const float4 pv = *reinterpret_cast<const float4*>(pw + j);
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          const int i = lane + k * ME_WAVE;
          if (DT || i < d) {
            const float4 vv = *reinterpret_cast<const float4*>(Vs + i * AS_VROW + j);
            acc[k] = fmaf(pv.x, vv.x, acc[k]);
            acc[k] = fmaf(pv.y, vv.y, acc[k]);
            acc[k] = fmaf(pv.z, vv.z, acc[k]);
            acc[k] = fmaf(pv.w, vv.w, acc[k]);
          }
        }
      }
      for (; j <= j_hi; ++j) {
        const float pj = pw[j];
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
          const int i = lane + k * ME_WAVE;
          if (DT || i < d) acc[k] = fmaf(pj, Vs[i * AS_VROW + j], acc[k]);
        }
      }
    }
    if (active) {
      ag_merge<KMAX>(mt, lt, acct, m, l, acc);  // the last chunk
      float* orow = out + ((size_t)t * nh + head) * d;
      const float inv = 1.f / lt;
#pragma unroll
      for (int k = 0; k < KMAX; ++k) {
        const int i = lane + k * ME_WAVE;
        if (DT || i < d) orow[i] = acct[k] * inv;
      }
    }
    seg = seg_end;
  }
}

// `items`: how many items the step's tokens belong to (0: unknown). Steps with two and more tokens per item on
// average go to the kernel that shares the tiles of keys and values among the tokens of a block; the results are
// the same bits either way.
//
// dv: size of the value heads (out is [tokens, nh * dv]); keep_first: the first keys that stay visible behind the window;
// unturn (float32 [positions, 2, dv/2] or null) and un_pairing (0: element j with j + dv/2; 1: 2j with 2j + 1): the
// angles that every output row is turned back by. Steps with any of these go to the first kernel.
//
// sink (float32 [nh] or null): a learned logit per head that counts once in the softmax's denominator and has no value (it
// is not multiplied by the scale). gate (or null; gate[t * gate_row + head] in the activations' type): every head's output
// is multiplied by the sigmoid of its gate before it is rounded.
// k_pool, v_pool, pool: pages of pooled blocks (entry b at page table[b / bs], slot b % bs: the mean of the keys and of the
// values at the positions b pool .. b pool + pool - 1) that are visible, beside the window's keys, once the window has passed
// them wholly; they share the softmax with the window's keys. out_row, out_col: the result's rows are out_row elements apart
// (0: nh * dv) and begin at column out_col; out_scale multiplies the result before it is rounded.
// softcap > 0: every scaled score s becomes softcap * tanh(s / softcap) before the softmax.
extern "C" int me_attention_general_capped(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                           const int* token_item, const int* block_table, int table_width, void* out,
                                           int num_tokens, int nh, int nkv, int d, int dv, int bs, int window, int keep_first,
                                           const float* unturn, int un_pairing, float scale, const float* sink, const void* gate,
                                           long long gate_row, const void* k_pool, const void* v_pool, int pool, long long out_row,
                                           int out_col, float out_scale, float softcap, int dtype, int items, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (pool < 0 || (pool > 0 && (window <= 0 || keep_first > 0 || !k_pool || !v_pool)))
    return me_fail("me_attention_general: pooled blocks of %d keys need a window, pages of their own and no kept first keys", pool);
  if (out_col < 0 || (out_row > 0 && out_col + (long long)nh * dv > out_row))
    return me_fail("me_attention_general: the result at column %d of a row of %lld", out_col, out_row);
  if (d <= 0 || d > AG_MAX_D_WIDE) return me_fail("me_attention_general: head_dim=%d must be in 1..%d", d, AG_MAX_D_WIDE);
  if (dv <= 0 || dv > AG_MAX_D_WIDE) return me_fail("me_attention_general: value head size %d must be in 1..%d", dv, AG_MAX_D_WIDE);
  const bool big = d > AG_MAX_D || dv > AG_MAX_D;  // the instance with eight elements a lane
  if (keep_first < 0 || (keep_first > 0 && window <= 0))
    return me_fail("me_attention_general: keep_first=%d needs a window", keep_first);
  if (unturn && (dv % 2 || (un_pairing & ~1))) return me_fail("me_attention_general: values of size %d, pairing %d", dv, un_pairing);
  const bool plain = dv == d && keep_first == 0 && !unturn && !sink && !gate && !big && pool == 0 && out_row <= 0 && out_col == 0 &&
                     out_scale == 1.f && !(softcap > 0.f);
  if (nh <= 0 || nkv <= 0 || nh % nkv)
    return me_fail("me_attention_general: %d query heads are not a multiple of %d key/value heads", nh, nkv);
  if (bs <= 0 || table_width <= 0 || window < 0)
    return me_fail("me_attention_general: block_size=%d table_width=%d window=%d", bs, table_width, window);
  const int group = nh / nkv;
  if (plain && dtype == ME_F32 && items > 0 && num_tokens >= 2 * items && d % 4 == 0 && bs % 4 == 0 && group <= 16 &&
      (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0) {
    const int tq = 16 / group > 0 ? 16 / group : 1, waves = tq * group;
    const size_t lds = ((size_t)64 * (d + AS_KPAD) + (size_t)d * AS_VROW + (size_t)waves * (d + 64)) * sizeof(float);
    int bs_shift = -1;
    if ((bs & (bs - 1)) == 0)
      for (bs_shift = 0; (1 << bs_shift) < bs;) ++bs_shift;
    const dim3 grid((num_tokens + tq - 1) / tq, nkv);
#define ME_SHARED_LAUNCH(DT)                                                                                                     \
  do {                                                                                                                           \
    static size_t allowed = 0; /* grows to the most this head size has asked for */                                             \
    if (lds > allowed) {                                                                                                         \
      if (hipFuncSetAttribute((const void*)attention_shared_f32_kernel<DT>, hipFuncAttributeMaxDynamicSharedMemorySize,          \
                              (int)lds) != hipSuccess)                                                                           \
        return me_fail("me_attention_general: %zu bytes of block memory for head_dim=%d are refused", lds, d);                   \
      allowed = lds;                                                                                                             \
    }                                                                                                                            \
    attention_shared_f32_kernel<DT><<<grid, waves * 64, lds, stream>>>(                                                          \
        (const float*)q, (const float*)k_cache, (const float*)v_cache, positions, token_item, block_table, table_width,         \
        (float*)out, num_tokens, nh, nkv, d, bs, bs_shift, window, scale, tq);                                                   \
  } while (0)
    if (d == 64)
      ME_SHARED_LAUNCH(64);
    else if (d == 128)
      ME_SHARED_LAUNCH(128);
    else if (d == 256)
      ME_SHARED_LAUNCH(256);
    else
      ME_SHARED_LAUNCH(0);
#undef ME_SHARED_LAUNCH
    return me_check_launch("me_attention_general");
  }
  const long long units = (long long)num_tokens * nh;
  // few units (decode steps): a block of eight waves each, which share a token's chunks of keys; else four units a block
  const int wpu = units < 2048 ? 8 : 1, waves = units < 2048 ? 8 : 4;
  const unsigned blocks = (unsigned)((units + waves / wpu - 1) / (waves / wpu));
#define ME_AG_LAUNCH(TT, KK)                                                                                                   \
  attention_general_kernel<TT, KK><<<blocks, waves * 64, 0, stream>>>(                                                         \
      (const TT*)q, (const TT*)k_cache, (const TT*)v_cache, positions, token_item, block_table, table_width, (TT*)out, num_tokens, \
      nh, nkv, d, dv, bs, window, keep_first, unturn, un_pairing, scale, wpu, sink, (const TT*)gate, (size_t)gate_row,             \
      (const TT*)k_pool, (const TT*)v_pool, pool, out_row > 0 ? out_row : (long long)nh * dv, out_col, out_scale, softcap)
  if (dtype == ME_F32) {
    if (big)
      ME_AG_LAUNCH(float, AG_MAX_D_WIDE / ME_WAVE);
    else
      ME_AG_LAUNCH(float, AG_MAX_D / ME_WAVE);
  } else {
    if (big)
      ME_AG_LAUNCH(bf16_t, AG_MAX_D_WIDE / ME_WAVE);
    else
      ME_AG_LAUNCH(bf16_t, AG_MAX_D / ME_WAVE);
  }
#undef ME_AG_LAUNCH
  return me_check_launch("me_attention_general");
}

extern "C" int me_attention_general_pooled(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                           const int* token_item, const int* block_table, int table_width, void* out,
                                           int num_tokens, int nh, int nkv, int d, int dv, int bs, int window, int keep_first,
                                           const float* unturn, int un_pairing, float scale, const float* sink, const void* gate,
                                           long long gate_row, const void* k_pool, const void* v_pool, int pool, long long out_row,
                                           int out_col, float out_scale, int dtype, int items, hipStream_t stream) {
  return me_attention_general_capped(q, k_cache, v_cache, positions, token_item, block_table, table_width, out, num_tokens, nh, nkv,
                                     d, dv, bs, window, keep_first, unturn, un_pairing, scale, sink, gate, gate_row, k_pool, v_pool,
                                     pool, out_row, out_col, out_scale, 0.f, dtype, items, stream);
}

extern "C" int me_attention_general_gated(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                          const int* token_item, const int* block_table, int table_width, void* out,
                                          int num_tokens, int nh, int nkv, int d, int dv, int bs, int window, int keep_first,
                                          const float* unturn, int un_pairing, float scale, const float* sink, const void* gate,
                                          long long gate_row, int dtype, int items, hipStream_t stream) {
  return me_attention_general_pooled(q, k_cache, v_cache, positions, token_item, block_table, table_width, out, num_tokens, nh, nkv,
                                     d, dv, bs, window, keep_first, unturn, un_pairing, scale, sink, gate, gate_row, nullptr, nullptr,
                                     0, 0, 0, 1.f, dtype, items, stream);
}

extern "C" int me_attention_general_ext(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                        const int* token_item, const int* block_table, int table_width, void* out,
                                        int num_tokens, int nh, int nkv, int d, int dv, int bs, int window, int keep_first,
                                        const float* unturn, int un_pairing, float scale, int dtype, int items,
                                        hipStream_t stream) {
  return me_attention_general_gated(q, k_cache, v_cache, positions, token_item, block_table, table_width, out, num_tokens, nh, nkv,
                                    d, dv, bs, window, keep_first, unturn, un_pairing, scale, nullptr, nullptr, 0, dtype, items,
                                    stream);
}

extern "C" int me_attention_general(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                                    const int* token_item, const int* block_table, int table_width, void* out,
                                    int num_tokens, int nh, int nkv, int d, int bs, int window, float scale,
                                    int dtype, int items, hipStream_t stream) {
  return me_attention_general_ext(q, k_cache, v_cache, positions, token_item, block_table, table_width, out, num_tokens, nh, nkv,
                                  d, d, bs, window, 0, nullptr, 0, scale, dtype, items, stream);
}
