// Running a step program: the choice of kernel per operation and step size, and the launches.
#include "program.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <mutex>
#include <set>
#include <tuple>

#include "../kernels.h"
#include "choice.h"

int me_fail(const char* fmt, ...);

namespace me {

namespace {

constexpr int kF32 = 0, kBF16 = 1;
constexpr int kDecodeWaves = 1024;  // waves that a decode attention launch aims at (four per compute unit of 256)

void ok(int code) {
  if (code) throw Error(kBadState, me_last_error());
}

struct Arena {
  char* base;
  size_t size, used = 0;
  void* take(size_t bytes) {
    const size_t at = (used + 255) & ~(size_t)255;
    if (at + bytes > size)
      throw Error(kBadState, "the step needs more workspace than the program's arena holds (" + std::to_string(at + bytes) +
                                 " of " + std::to_string(size) + " bytes)");
    used = at + bytes;
    return base + at;
  }
};

struct Pending {
  const void* delta = nullptr;
  const float* parts = nullptr;
  int num_parts = 0;
  long long stride = 0;
  // A delta that has added itself to the stream and left the norm behind it half done: bf16(x * w) in the buffer of
  // normed rows and the rows' sums of squares in `ss_blocks` partial sums, for the product behind the norm `carried_w`.
  const float* ss = nullptr;
  int ss_blocks = 0;
  const void* carried_w = nullptr;
  float scale = 1.f;  // what the block multiplies the delta by when it is added to the stream
  bool any() const { return delta || parts; }
  bool carried() const { return ss != nullptr; }
};

int compute_units() {
  static int units = 0;
  if (!units) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      units = n;
    else
      units = 256;
  }
  return units;
}

std::mutex g_refused_mutex;
std::set<std::tuple<int, int, int>> g_refused;  // (N, K, output type) the GEMM library has no algorithm for

// A plain bfloat16 product of many rows: the GEMM library, as the reference hands every projection to one;
// sizes it has no algorithm for go to the kernels of this folder.
void library_product(const void* x, const void* w, void* out, int m, int n, int k, int out_dtype, hipStream_t stream) {
  const auto shape = std::make_tuple(n, k, out_dtype);
  bool refused;
  {
    std::lock_guard<std::mutex> hold(g_refused_mutex);
    refused = g_refused.count(shape) != 0;
  }
  if (!refused) {
    if (me_gemm_bf16_library(x, w, out, m, n, k, out_dtype, stream) == 0) return;
    std::lock_guard<std::mutex> hold(g_refused_mutex);
    g_refused.insert(shape);
  }
  if (k % 64 == 0 && m > kSmallMaxRows && (((uintptr_t)x | (uintptr_t)w) & 15) == 0) {  // the tiled matrix-core kernel of this folder
    ok(me_gemm_bf16_tiled(x, w, out, m, n, k, 0, out_dtype, 0, stream));
    return;
  }
  if (k % 8 == 0) {  // slices of 64 rows through the small matrix-core kernel
    const size_t out_elem = out_dtype == kF32 ? 4 : 2;
    for (int lo = 0; lo < m; lo += kSmallMaxRows) {
      const int rows = std::min(kSmallMaxRows, m - lo);
      ok(me_gemm_bf16_small((const char*)x + (size_t)lo * k * 2, nullptr, nullptr, nullptr, 0.f, nullptr, w,
                            (char*)out + (size_t)lo * n * out_elem, rows, n, k, 0, 0, out_dtype, 1, stream));
    }
    return;
  }
  ok(me_gemm_plain(x, w, out, m, n, k, kBF16, out_dtype, stream));
}

// x += a . w^T through the library; false (and nothing done) for sizes it has no algorithm for.
bool library_adds(const void* a, const void* w, float* x, int m, int n, int k, hipStream_t stream) {
  const auto shape = std::make_tuple(n, k, kF32);
  {
    std::lock_guard<std::mutex> hold(g_refused_mutex);
    if (g_refused.count(shape)) return false;
  }
  if (me_gemm_bf16_library_add(a, w, x, m, n, k, stream) == 0) return true;
  std::lock_guard<std::mutex> hold(g_refused_mutex);
  g_refused.insert(shape);
  return false;
}

// (keys per split, number of splits) of a decode launch: enough waves to fill the chip, splits of at least 64
// keys, whole tiles of 16 (rounded to 64 keys, 3 items at a context of 4,096 had 32 splits of 128 keys where 43 of 96
// fit: a step of 3 / 5 / 9 items 1.348 -> 1.293 / 1.501 -> 1.452 / 1.818 -> 1.772 ms, other counts level).
void decode_splits(int items, int kv_units, int max_ctx, int& split_keys, int& num_splits) {
  const int units = std::max(1, items * kv_units);
  const int splits = std::max(1, std::min((kDecodeWaves + units - 1) / units, std::max(max_ctx, 64) / 64));
  split_keys = (max_ctx + splits - 1) / splits;
  split_keys = (split_keys + 15) / 16 * 16;
  num_splits = (max_ctx + split_keys - 1) / split_keys;
}

struct SplitPlan {
  int split_keys, num_splits, full_splits;
  const int* live;
};

// The grid of a launch that a graph replays with fewer live items than it holds is laid out for the fewest it
// will ever see; the kernel reads the count of live items and takes as many of the grid's splits as they need.
SplitPlan split_plan(int items, int kv_units, int max_ctx, int least_live, const int* live_count) {
  int keys, full;
  decode_splits(items, kv_units, max_ctx, keys, full);
  if (!live_count || least_live >= items) return {keys, full, full, nullptr};
  int splits;
  decode_splits(std::max(1, least_live), kv_units, max_ctx, keys, splits);
  return {keys, splits, std::min(full, splits), live_count};
}

// An attention operation that the kernels of the plain form serve: keys and values of one size, a window without kept
// first keys, rotation of halves, values as they are.
bool attention_is_plain(const Op& op) {
  return (op.i[9] == 0 || op.i[9] == op.i[2]) && op.i[10] == 0 && op.i[11] == 0 && op.i[12] == 0 && op.i[13] == 0 && op.i[14] == 0;
}

// A latent attention operation: the rows of its value pages (i8; 0: the latent's rank), and whether the matrix-core attention
// kernels serve it: bfloat16, value pages that hold the whole key (the kernels take keys and values of one size), a key
// size they are built for, at most 16 heads (all of them share the one key/value head).
int latent_value_rows(const Op& op) { return op.i[8] ? (int)op.i[8] : (int)op.i[3]; }
bool latent_takes_matrix_cores(const Op& op, int dtype) {
  const int dk = (int)(op.i[3] + op.i[2]);
  return dtype == kBF16 && latent_value_rows(op) == dk && me_attention_mfma_supported(dk, (int)op.i[5]) && op.i[0] <= 16;
}

// How many residual streams the tokens of a program have (kOpStreams; 1 without).
int streams_of(const std::vector<Op>& ops) {
  int s = 1;
  for (const Op& op : ops)
    if (op.kind == kOpStreams) s = std::max(s, (int)op.i[0]);
  return s;
}

// Whether prompts of an attention operation beyond the plain form go to the tiled matrix-core kernel: bfloat16, keys and
// values of one size that the kernel is built for, up to 16 heads to a key/value head.
bool attention_takes_tiled_prefill(const Op& op, int dtype) {
  const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2], bs = (int)op.i[4];
  return dtype == kBF16 && (op.i[9] == 0 || op.i[9] == d) && me_attention_mfma_supported(d, bs) && nh / nkv <= 16;
}

// Whether an attention operation over a window and pooled blocks goes to the matrix-core kernels: bfloat16, keys and values of
// one size that the kernels are built for, up to 16 heads to a key/value head, results at rows and a column that are multiples of 4.
bool pooled_takes_matrix_cores(const Op& op, int dtype, long long out_row) {
  const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2], dv = (int)op.i[3], bs = (int)op.i[4];
  // (pooled blocks lie before a window; without them the kernels take every window, none, a sink and bounded scores)
  return dtype == kBF16 && dv == d && (op.i[5] > 0 || op.i[6] == 0) && me_attention_mfma_supported(d, bs) && nh / nkv <= 16 &&
         out_row % 4 == 0 && op.i[11] % 4 == 0;
}

int groups_of(int64_t v) { return v > 1 ? (int)v : 1; }
bool act_code_is_ungated(int code) { return code >= 16; }  // csrc/common.h: MeAct
constexpr int kTimeMixStackedTokens = 32;  // up to here time mixing's five products are one (Run::time_mix)
float scale_of(float f) { return f == 0.f ? 1.f : f; }

class Run {
 public:
  Run(const Program& prog, const std::vector<Value>& values, const StepView& s, Arena& arena, int32_t* fed_tokens,
      hipStream_t stream)
      : prog_(prog), values_(values), s_(s), arena_(arena), fed_tokens_(fed_tokens), stream_(stream), dtype_(prog.dtype()),
        elem_(prog.dtype() == kF32 ? 4 : 2), t_(s.lay.tokens), h_(prog.hidden()), streams_(streams_of(prog.ops())) {
    x_ = (float*)arena_.take((size_t)streams_ * t_ * h_ * 4);  // (several streams: [streams, tokens, hidden], x_ is the first)
    spare_ = (float*)arena_.take((size_t)streams_ * t_ * h_ * 4);
    normed_ = arena_.take((size_t)t_ * h_ * elem_);
    for (const Value& v : values) bufs_.push_back(arena_.take((size_t)t_ * v.cols * v.elem));
  }

  RunResult go() {
    const std::vector<Op>& ops = prog_.ops();
    for (size_t at = 0; at < ops.size(); ++at) {
      const Op& op = ops[at];
      next_ = at + 1 < ops.size() ? &ops[at + 1] : nullptr;
      const size_t mark = arena_.used;
      released_to_ = (size_t)-1;
      if (pending_.carried() && op.kind != kOpNormLinear)
        throw Error(kBroken, "a norm was left to a product that does not follow");
      step(op);
      // the logits, the drawn tokens and partial sums that wait for the next norm outlive their operation;
      // an operation that used up waiting partial sums gives their memory back too
      if (op.kind != kOpHead && op.kind != kOpHeadRows && op.kind != kOpStreamHead && op.kind != kOpSample && op.kind != kOpLinearDelta)
        arena_.used = released_to_ != (size_t)-1 ? released_to_ : mark;
    }
    return result_;
  }

 private:
  const int32_t* idx(int offset) const { return s_.dev + offset; }

  void step(const Op& op) {
    switch (op.kind) {
      case kOpEmbed: {
        const int table_dtype = dtype_;
        if (s_.fed && fed_tokens_)
          ok(me_embed_fed(x_, op.p[0], idx(s_.lay.token_ids), idx(s_.lay.token_source), fed_tokens_, t_, h_, prog_.vocab(),
                          op.f[0], table_dtype, stream_));
        else
          ok(me_embed(x_, op.p[0], idx(s_.lay.token_ids), t_, h_, prog_.vocab(), op.f[0], table_dtype, stream_));
        pending_ = Pending();
        break;
      }
      case kOpNormLinear:
        norm_linear(op);
        break;
      case kOpNorm:
        if (op.i[1]) {  // a second norm of the same stream: nothing is added, what was set aside stays aside
          if (pending_.any() || pending_.carried()) throw Error(kBroken, "a result is pending before a second norm of the stream");
          ok(me_add_group_rmsnorm2(x_, nullptr, nullptr, 0, 0, nullptr, nullptr, 0, 0, 1.f, (const float*)op.p[0], bufs_[op.out], nullptr,
                                   t_, h_, groups_of(op.i[0]), op.f[0], 0, dtype_, stream_));
          break;
        }
        add_norm((const float*)op.p[0], op.f[0], bufs_[op.out], groups_of(op.i[0]));
        break;
      case kOpPooledAttention:
        pooled_attention(op);
        break;
      case kOpDeltaRule:
        delta_rule(op);
        break;
      case kOpLinear:
        product(bufs_[op.in], op.p[1], (int)op.i[0], (int)op.i[1], (int)op.i[2], dtype_, bufs_[op.out]);
        break;
      case kOpLinearDelta:
        linear_delta(op);
        break;
      case kOpDelta:
        pending_ = Pending();
        pending_.delta = bufs_[op.in];
        pending_.scale = scale_of(op.f[0]);
        break;
      case kOpDecayState:
        decay_state(op);
        break;
      case kOpHold:
        if (held_.any()) throw Error(kBroken, "two results are set aside at once");
        if (pending_.carried()) throw Error(kBroken, "a result that added itself cannot be set aside");
        held_ = pending_;
        held_mark_ = parts_mark_;
        parts_mark_ = (size_t)-1;
        pending_ = Pending();
        break;
      case kOpAttention:
        attention(op);
        break;
      case kOpHead:
        head(op);
        break;
      case kOpSample:
        sample();
        break;
      case kOpAdd:
        add_held();
        if (pending_.any() && pending_.scale != 1.f)
          ok(me_residual_add_scaled(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, pending_.scale, t_, h_,
                                    dtype_, stream_));
        else if (pending_.any())
          ok(me_residual_add(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, t_, h_, dtype_, stream_));
        pending_ = Pending();
        release_parts();
        break;
      case kOpCall:
        call(op);
        break;
      case kOpHeadRows:
        head_rows(op);
        break;
      case kOpStreams:
        if (pending_.any() || held_.any() || pending_.carried()) throw Error(kBroken, "a result is pending where the streams begin");
        ok(me_streams_spread(x_, (long long)t_ * h_, streams_, stream_));
        spread_ = true;
        break;
      case kOpStreamNorm:
        stream_norm(op, bufs_[op.out], nullptr, t_, 1);
        break;
      case kOpStreamHead:
        stream_head(op);
        break;
      case kOpStreamNormLinear:
        stream_norm_linear(op);
        break;
      case kOpLatentAttention:
        latent_attention(op);
        break;
      case kOpRoutedFF:
        routed_ff(op);
        break;
      case kOpResultNorm:
        result_norm(op);
        break;
      case kOpTokenGate: {
        const bool fed = s_.fed && fed_tokens_;
        ok(me_token_gate(bufs_[op.in], op.p[0], idx(s_.lay.token_ids), fed ? idx(s_.lay.token_source) : nullptr, fed ? fed_tokens_ : nullptr,
                         bufs_[op.out], t_, (int)values_[op.in].cols, op.i[1], (int)op.i[0], prog_.vocab(), (int)op.i[2], dtype_, stream_));
        break;
      }
      case kOpActivate:
        ok(me_act_rows(bufs_[op.in], bufs_[op.out], (long long)t_ * values_[op.in].cols, (int)op.i[0], dtype_, stream_));
        break;
      case kOpTimeMix:
        time_mix(op);
        break;
      default:
        throw Error(kBadValue, "unknown operation in a step program");
    }
  }

  // x += pending; out = rmsnorm(x) * w, as a kernel of its own.
  // A result that was set aside, where the kernel at hand takes one delta only: into the stream by a kernel of its own.
  void add_held() {
    if (!held_.any()) return;
    ok(me_residual_add_scaled(x_, held_.delta, held_.parts, held_.num_parts, held_.stride, held_.scale, t_, h_, dtype_, stream_));
    held_ = Pending();
  }

  void add_norm(const float* w, float eps, void* out, int groups = 1) {
    if (held_.any() && held_.scale != pending_.scale && pending_.any()) add_held();
    if (groups > 1 || pending_.scale != 1.f || held_.any()) {  // a norm in groups, a block that multiplies what its parts give,
                                                              // or two parts' results at once
      const float scale = pending_.any() ? pending_.scale : held_.scale;
      ok(me_add_group_rmsnorm2(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, held_.delta, held_.parts,
                               held_.num_parts, held_.stride, scale, w, out, nullptr, t_, h_, groups, eps, 1, dtype_, stream_));
      held_ = Pending();
    } else
      ok(me_add_rmsnorm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, w, out, nullptr, t_, h_, eps, 1,
                        dtype_, stream_));
    pending_ = Pending();
    release_parts();
  }

  // x += scale * rmsnorm(pending) * w; out = x in the compute dtype (a block that norms its sublayers' results).
  void result_norm(const Op& op) {
    if (held_.any() || pending_.carried()) throw Error(kBroken, "a result was set aside or added itself before the norm of a sublayer's result");
    if (pending_.any() && !op.p[0]) throw Error(kBadValue, "a sublayer's result without a norm weight");
    ok(me_result_norm_add(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, (const float*)op.p[0],
                          op.out >= 0 ? bufs_[op.out] : nullptr, t_, h_, op.f[0], pending_.scale, dtype_, stream_));
    pending_ = Pending();
    release_parts();
  }

  // Time mixing: blends of neighbouring tokens, five products, the decay, the scan over the items' tokens, norm and gate.
  void time_mix(const Op& op) {
    const int heads = (int)op.i[0], d = (int)op.i[1], rank = (int)op.i[2], n = heads * d;
    const long long state_row = op.i[4], prev_at = op.i[5];
    if (op.p[11] && t_ <= kTimeMixStackedTokens) {
      // Few tokens (decode steps): the five blends of a token are five rows of ONE product with the five weights stacked. A row meets
      // all of the stacked weight, of which its own fifth is used: five times the multiply-adds, but the weights are read once and the
      // step waits for one product, not five (at these sizes a product is the time its weights take to arrive).
      const long long wide = 4ll * n + rank;
      char* x5 = (char*)arena_.take((size_t)5 * t_ * h_ * elem_);
      char* p5 = (char*)arena_.take((size_t)5 * t_ * wide * elem_);
      void* ws = arena_.take((size_t)me_time_mix_workspace(t_, heads, d));
      void* rows[5];
      for (int i = 0; i < 5; ++i) rows[i] = x5 + (size_t)i * h_ * elem_;
      ok(me_time_shift(bufs_[op.in], (float*)op.p[7], state_row, prev_at, idx(s_.lay.state_slots), idx(s_.lay.item_start), idx(s_.lay.token_item),
                       idx(s_.lay.positions), (const float*)op.p[0], rows, 5ll * h_, t_, s_.lay.items, h_, dtype_, stream_));
      product(x5, op.p[11], (int)wide, h_, 0, dtype_, p5, kRolePlain, 5 * t_);
      auto at = [&](int i) { return p5 + ((size_t)i * wide + (size_t)i * n) * elem_; };  // blend i's row of a token, at its own columns
      ok(me_time_mix(at(0), at(1), at(2), at(3), at(4), op.p[3], (const float*)op.p[4], (const float*)op.p[5], (const float*)op.p[6],
                     (float*)op.p[7], state_row, idx(s_.lay.state_slots), idx(s_.lay.item_start), bufs_[op.out], values_[op.out].cols, (int)op.i[3],
                     op.f[1], t_, s_.lay.items, heads, d, rank, op.f[0], 5 * wide, dtype_, ws, stream_));
      return;
    }
    void* mixes[5];
    for (int i = 0; i < 5; ++i) mixes[i] = arena_.take((size_t)t_ * h_ * elem_);
    void* proj[4];
    for (int i = 0; i < 4; ++i) proj[i] = arena_.take((size_t)t_ * n * elem_);
    void* z = arena_.take((size_t)t_ * rank * elem_);
    void* ws = arena_.take((size_t)me_time_mix_workspace(t_, heads, d));
    ok(me_time_shift(bufs_[op.in], (float*)op.p[7], state_row, prev_at, idx(s_.lay.state_slots), idx(s_.lay.item_start), idx(s_.lay.token_item),
                     idx(s_.lay.positions), (const float*)op.p[0], mixes, h_, t_, s_.lay.items, h_, dtype_, stream_));
    const void* weights[4] = {op.p[1], op.p[8], op.p[9], op.p[10]};  // r, k, v, gate
    for (int i = 0; i < 4; ++i) product(mixes[i], weights[i], n, h_, 0, dtype_, proj[i]);
    product(mixes[4], op.p[2], rank, h_, 0, dtype_, z);
    ok(me_time_mix(proj[0], proj[1], proj[2], proj[3], z, op.p[3], (const float*)op.p[4], (const float*)op.p[5], (const float*)op.p[6],
                   (float*)op.p[7], state_row, idx(s_.lay.state_slots), idx(s_.lay.item_start), bufs_[op.out], values_[op.out].cols, (int)op.i[3],
                   op.f[1], t_, s_.lay.items, heads, d, rank, op.f[0], 0, dtype_, ws, stream_));
  }

  void release_parts() {
    if (held_.any()) return;  // (what was set aside lies below the pending result's memory: both go together)
    if (held_mark_ != (size_t)-1 && !pending_.parts && !pending_.ss) {
      arena_.used = released_to_ = std::min(held_mark_, parts_mark_);
      held_mark_ = parts_mark_ = (size_t)-1;
      return;
    }
    if (parts_mark_ != (size_t)-1 && !pending_.parts && !pending_.ss) {
      arena_.used = released_to_ = parts_mark_;
      parts_mark_ = (size_t)-1;
    }
  }

  void norm_linear(const Op& op) {
    const float* w_norm = (const float*)op.p[0];
    const int rows_of_w = (int)op.i[0], k = (int)op.i[1];
    const int gated = (int)op.i[2];  // 0, or the code of the gate's activation
    if (k != h_) throw Error(kBadValue, "a product behind a norm reads the hidden size");
    const int n = gated ? rows_of_w / 2 : rows_of_w;
    if (pending_.carried()) {  // the add is done and the norm half done: this product multiplies its rows by the rest
      if (op.p[0] != pending_.carried_w) throw Error(kBroken, "a norm was left to the product behind another norm");
      const ProductChoice c = choose_product(dtype_, kRolePlain, t_, rows_of_w, k, gated, dtype_, compute_units(), true);
      if (c.kernel == kProductSmall && !c.gate_after)
        ok(me_gemm_bf16_small_scaled(normed_, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, pending_.ss, pending_.ss_blocks, k,
                                     op.f[0], stream_));
      else if (c.kernel == kProductStream && !c.gate_after)
        ok(me_gemm_bf16_stream_scaled(normed_, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, compute_units(), pending_.ss,
                                      pending_.ss_blocks, k, op.f[0], stream_));
      else
        throw Error(kBroken, "a norm was left to a product whose kernel does not scale its rows");
      pending_ = Pending();
      release_parts();
      return;
    }
    if (groups_of(op.i[3]) > 1 || pending_.scale != 1.f || held_.any()) {  // no product of this folder carries such a norm as its prologue
      add_norm(w_norm, op.f[0], normed_, groups_of(op.i[3]));
      product(normed_, op.p[1], rows_of_w, k, gated, dtype_, bufs_[op.out]);
      return;
    }
    const int pending = pending_.parts ? kPendingParts : pending_.delta ? kPendingTensor : kPendingNone;
    // Where the add and the norm ride on the product the sum goes to the second residual buffer, since other blocks
    // of the kernel still read the first.
    switch (choose_norm_fusion(dtype_, t_, rows_of_w, k, pending, compute_units(), true)) {
      case kNormInStream: {
        const bool adds = pending_.any();
        ok(me_gemm_bf16_stream_norm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, w_norm, op.f[0],
                                    adds ? spare_ : nullptr, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, compute_units(),
                                    stream_));
        if (adds) std::swap(x_, spare_);
        pending_ = Pending();
        release_parts();
        return;
      }
      case kNormInSmall:
        ok(me_gemm_bf16_small(nullptr, x_, pending_.delta, w_norm, op.f[0], pending_.delta ? spare_ : nullptr, op.p[1],
                              bufs_[op.out], t_, n, k, 1, gated, dtype_, 1, stream_));
        if (pending_.delta) std::swap(x_, spare_);
        pending_ = Pending();
        return;
      default:
        add_norm(w_norm, op.f[0], normed_);
        product(normed_, op.p[1], rows_of_w, k, gated, dtype_, bufs_[op.out]);
    }
  }

  // out = x . W^T (gated, the code of an activation: act(gate) * up with W = [gate rows; up rows]), by the kernel
  // that choose_product names.
  void product(const void* x, const void* w, int rows_of_w, int k, int gated, int out_dtype, void* out, int role = kRolePlain,
               int rows = -1) {
    const int m = rows < 0 ? t_ : rows;
    const int n = gated ? rows_of_w / 2 : rows_of_w;
    const ProductChoice c = choose_product(dtype_, role, m, rows_of_w, k, gated, out_dtype, compute_units(), true);
    void* dst = out;
    const int cols = c.gate_after ? rows_of_w : n;
    const int inner_dtype = c.gate_after ? dtype_ : out_dtype;
    if (c.gate_after) dst = arena_.take((size_t)m * rows_of_w * elem_);
    const int epilogue = c.gate_after ? 0 : gated;
    switch (c.kernel) {
      case kProductF32:
        ok(me_gemm_f32((const float*)x, (const float*)w, (float*)dst, m, cols, k, stream_));
        break;
      case kProductSmall:
        ok(me_gemm_bf16_small(x, nullptr, nullptr, nullptr, 0.f, nullptr, w, dst, m, cols, k, 0, epilogue, inner_dtype, 1, stream_));
        break;
      case kProductStream:
        ok(me_gemm_bf16_stream(x, w, dst, m, cols, k, epilogue, c.partial_sums ? kF32 : inner_dtype, c.runs, compute_units(),
                               stream_));
        break;
      case kProductTiled:
        ok(me_gemm_bf16_tiled(x, w, dst, m, cols, k, epilogue, inner_dtype, 0, stream_));
        break;
      default:
        library_product(x, w, dst, m, cols, k, c.partial_sums ? kF32 : inner_dtype, stream_);
    }
    if (c.gate_after) ok(me_swiglu(dst, out, m, n, gated, dtype_, stream_));
  }

  // A product whose result only ever is the pending delta of the residual stream.
  void linear_delta(const Op& op) {
    const int n = (int)op.i[0], k = (int)op.i[1];
    if (n != h_) throw Error(kBadValue, "a delta of the residual stream has the hidden size");
    const void* x = bufs_[op.in];
    const float scale = scale_of(op.f[0]);
    const bool stays = op.i[2] != 0 || spread_;  // the result waits for whatever rewrites the stream(s) behind it
    pending_ = Pending();
    pending_.scale = scale;
    if (attn_parts_.o) {  // decode attention left its splits to this product
      const AttnParts a = attn_parts_;
      attn_parts_ = AttnParts();
      if (a.value != op.in || k != a.nh * a.d) throw Error(kBroken, "attention left its splits to a product that does not follow");
      const int runs = me_attention_out_product_runs(a.nh);
      parts_mark_ = a.mark;
      float* parts = (float*)arena_.take((size_t)runs * t_ * n * 4);
      ok(me_attention_out_product_bf16(a.o, a.ml, a.splits, op.p[1], parts, t_, a.nh, a.d, n, stream_));
      pending_.parts = parts;
      pending_.num_parts = runs;
      pending_.stride = (long long)t_ * n;
      return;
    }
    if (!stays && scale == 1.f && !held_.any() && next_ && next_->kind == kOpNormLinear && next_->i[1] == h_ && groups_of(next_->i[3]) == 1 &&
        choose_carried_norm(dtype_, t_, n, k, (int)next_->i[0], (int)next_->i[2], compute_units(), true)) {
      // x += product in the product's epilogue, which also starts the norm behind it (choice.cpp)
      const int blocks = me_gemm_bf16_stream_carry_blocks(t_, n, k, compute_units());
      parts_mark_ = arena_.used;
      float* ss = (float*)arena_.take((size_t)t_ * blocks * 4);
      ok(me_gemm_bf16_stream_carry(x, op.p[1], x_, normed_, ss, (const float*)next_->p[0], t_, n, k, compute_units(), stream_));
      pending_.ss = ss;
      pending_.ss_blocks = blocks;
      pending_.carried_w = next_->p[0];
      return;
    }
    const ProductChoice c = choose_product(dtype_, kRoleDeltaInto, t_, n, k, 0, dtype_, compute_units(), true);
    if (c.adds_into) {  // x += product, in the library's epilogue: nothing stays pending
      if (!stays && scale == 1.f && library_adds(x, op.p[1], x_, t_, n, k, stream_)) {  // (a result set aside waits for the next add as before)
        pending_ = Pending();
        return;
      }
      // (a size the library has no algorithm for: the product as one partial sum, through this folder's kernels)
      parts_mark_ = arena_.used;
      float* sum = (float*)arena_.take((size_t)t_ * n * 4);
      library_product(x, op.p[1], sum, t_, n, k, kF32, stream_);
      pending_.parts = sum;
      pending_.num_parts = 1;
      pending_.stride = (long long)t_ * n;
      return;
    }
    if (c.partial_sums) {  // float32 sums over runs of k (or one whole sum) that wait for the next add-and-norm
      parts_mark_ = arena_.used;
      float* parts = (float*)arena_.take((size_t)c.runs * t_ * n * 4);
      product(x, op.p[1], n, k, 0, kF32, parts, kRoleDelta);
      pending_.parts = parts;
      pending_.num_parts = c.runs;
      pending_.stride = (long long)t_ * n;
      return;
    }
    const size_t mark = arena_.used;
    product(x, op.p[1], n, k, 0, dtype_, bufs_[op.out], kRoleDelta);
    arena_.used = mark;
    pending_.delta = bufs_[op.out];
  }

  void attention(const Op& op) {
    const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2], rd = (int)op.i[3], bs = (int)op.i[4];
    const int window = (int)op.i[5], g = (int)op.i[7];
    const bool owns = op.i[6] != 0;
    const float eps = op.f[0], scale = op.f[1];
    const float* q_w = (const float*)op.p[0];
    const float* k_w = owns ? (const float*)op.p[1] : nullptr;
    const float* rope = (const float*)op.p[2];
    void *kc = (void*)op.p[3], *vc = (void*)op.p[4];
    if (g < 0 || g >= (int)s_.lay.widths.size()) throw Error(kBadValue, "an attention layer names a cache group the step lacks");
    const int32_t* table = idx(s_.lay.tables[g]);
    const int width = s_.lay.widths[g], items = s_.lay.items, group = nh / nkv;
    if (rope && op.i[8] < s_.max_ctx)
      throw Error(kBadValue, "the rotary table covers " + std::to_string(op.i[8]) + " positions, the step may reach " +
                                 std::to_string(s_.max_ctx));
    void* out = bufs_[op.out];
    const void* qkv = bufs_[op.in];
    if (!attention_is_plain(op)) {  // value heads of their own size, kept first keys, the other pairing, turned values
      const int dv = op.i[9] ? (int)op.i[9] : d, keep_first = (int)op.i[10], pairing = (int)op.i[11];
      const float* v_table = op.i[12] ? (const float*)op.p[5] : nullptr;
      const int v_pairing = op.i[12] ? (int)op.i[12] - 1 : 0;
      if (!owns) throw Error(kBadValue, "an attention layer of this form writes its own pages");
      void* q = arena_.take((size_t)t_ * nh * d * elem_);
      const bool gated = op.i[14] != 0;  // the rows end in a gate per head
      const long long row = (long long)(nh + nkv) * d + (long long)nkv * dv + (gated ? nh : 0);
      const char* gate = gated ? (const char*)qkv + (size_t)(row - nh) * elem_ : nullptr;
      int segments = 0;
      if (t_ >= 64 && dv == d && !gated)  // many tokens: the values are turned and written a page segment (a transposed tile) at a time
        for (int i = 0; i < items; ++i) segments += (s_.starts[i] + s_.qlens[i] - 1) / 16 - s_.starts[i] / 16 + 1;
      ok(me_qkv_rotate_scatter_rows(qkv, gated ? row : 0, q_w, k_w, rope, rd, pairing, v_table, v_pairing, op.f[2], (int)op.i[13],
                                    idx(s_.lay.positions), idx(s_.lay.token_item), table, width, q, kc, vc, t_, nh, nkv, d, dv, bs, eps,
                                    dtype_, segments ? idx(s_.lay.item_start) : nullptr, items, segments, stream_));
      if (s_.decode_only && attention_takes_tiled_prefill(op, dtype_)) {
        // one new token per item: the split-context kernel, which deals the kept first keys' tiles to its splits before
        // the window's; a second kernel (or the blocks themselves) adds up the splits
        if ((long long)width * bs < s_.max_ctx) throw Error(kBadValue, "the block table cannot hold the step's longest context");
        const SplitPlan sp = split_plan(items, nkv * ((group + 15) / 16), s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
        float* part_o = (float*)arena_.take((size_t)items * nh * sp.num_splits * d * 4);
        float* part_ml = (float*)arena_.take((size_t)items * nh * sp.num_splits * 2 * 4);
        ok(me_attention_decode_bf16_kept(q, kc, vc, idx(s_.lay.item_ctx), table, width, out, part_o, part_ml, items, nh, nkv, d, bs,
                                         window, keep_first, scale, sp.split_keys, sp.num_splits, s_.max_ctx, sp.live, sp.full_splits,
                                         kDecodeWaves, idx(s_.lay.live_items) + 1, stream_));
        if (v_table) ok(me_unturn_rows(out, v_table, v_pairing, idx(s_.lay.positions), t_, nh, dv, dtype_, stream_));
        if (gate) ok(me_head_gate(out, gate, row, t_, nh, dv, dtype_, stream_));
        return;
      }
      if (!s_.decode_only && attention_takes_tiled_prefill(op, dtype_)) {
        // prompts and portions in bfloat16 with keys and values of one size the matrix cores take: the tiled kernel, whose
        // work list has an entry of its own for the kept first keys; the outputs are turned back by a pass of their own
        auto it = s_.plans.find({nh, nkv, d, window, keep_first});
        if (it == s_.plans.end()) throw Error(kBroken, "the step has no work list for a prefill attention layer");
        const StepView::Plan& p = it->second;
        float *part_o = nullptr, *part_ml = nullptr;
        if (p.max_chunks > 1) {
          part_o = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * d * 4);
          part_ml = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * 2 * 4);
        }
        ok(me_attention_prefill_bf16_kept(q, kc, vc, items, table, width, out, idx(p.work), idx(p.bundle_first), p.bundles, part_o,
                                          part_ml, p.token_chunks >= 0 ? idx(p.token_chunks) : nullptr, p.max_chunks, t_, nh, nkv, d,
                                          bs, window, keep_first, scale, p.columns, stream_));
        if (v_table) ok(me_unturn_rows(out, v_table, v_pairing, idx(s_.lay.positions), t_, nh, dv, dtype_, stream_));
        if (gate) ok(me_head_gate(out, gate, row, t_, nh, dv, dtype_, stream_));
        return;
      }
      ok(me_attention_general_gated(q, kc, vc, idx(s_.lay.positions), idx(s_.lay.token_item), table, width, out, t_, nh, nkv, d, dv,
                                    bs, window, keep_first, v_table, v_pairing, scale, nullptr, gate, row, dtype_, items, stream_));
      return;
    }
    const bool mfma = dtype_ == kBF16 && me_attention_mfma_supported(d, bs) && group <= 16;
    const size_t mark = arena_.used;
    auto partials = [&](const SplitPlan& sp, float*& part_o, float*& part_ml) {
      part_o = (float*)arena_.take((size_t)items * nh * sp.num_splits * d * 4);
      part_ml = (float*)arena_.take((size_t)items * nh * sp.num_splits * 2 * 4);
    };
    // A decode step of very few items leaves the splits' partial results to the output projection behind it: no kernel
    // of its own adds them up.
    auto leaves_to_product = [&](const SplitPlan& sp, float* part_o, float* part_ml) {
      if (!(next_ && next_->kind == kOpLinearDelta && next_->in == op.out && next_->i[0] == h_ && next_->i[1] == (int64_t)nh * d &&
            items == t_ && choose_split_sum_in_product(dtype_, items, h_, true) &&
            me_attention_decode_leaves_parts(items, nh, nkv, d, sp.num_splits) &&
            me_attention_out_product_supported(items, nh, d, h_, sp.num_splits)))
        return false;
      attn_parts_.o = part_o;
      attn_parts_.ml = part_ml;
      attn_parts_.splits = sp.num_splits;
      attn_parts_.nh = nh;
      attn_parts_.d = d;
      attn_parts_.value = op.out;
      attn_parts_.mark = mark;
      released_to_ = arena_.used;  // the partial results outlive this operation
      return true;
    };
    const int chunks = (group + 15) / 16;
    if (s_.decode_only && (long long)width * bs < s_.max_ctx && mfma)
      throw Error(kBadValue, "the block table cannot hold the step's longest context");
    if (dtype_ == kBF16 && s_.decode_only && me_attention_decode_fused_supported(d, bs, rd, group)) {
      // one new token per item: norm, rotary, page write and attention in one launch
      const SplitPlan sp = split_plan(items, nkv * chunks, s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
      float *part_o, *part_ml;
      partials(sp, part_o, part_ml);
      if (leaves_to_product(sp, part_o, part_ml)) out = nullptr;
      ok(me_attention_decode_fused_bf16(qkv, q_w, k_w, rope, rd, eps, owns ? 1 : 0, kc, vc, idx(s_.lay.item_ctx), table, width, out,
                                        part_o, part_ml, items, nh, nkv, d, bs, window, scale, sp.split_keys, sp.num_splits,
                                        s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves, idx(s_.lay.live_items) + 1, stream_));
      return;
    }
    void* q = arena_.take((size_t)t_ * nh * d * elem_);
    int segments = 0, seg_items = 0;
    if (owns && t_ >= 64) {  // many tokens: the values are written a page segment (a transposed tile) at a time
      seg_items = items;
      for (int i = 0; i < items; ++i) segments += (s_.starts[i] + s_.qlens[i] - 1) / 16 - s_.starts[i] / 16 + 1;
    }
    ok(me_qk_norm_rope_scatter(qkv, q_w, k_w, rope, idx(s_.lay.positions), idx(s_.lay.token_item), table, width, q, kc, vc, t_, nh,
                               nkv, d, rd, bs, eps, owns ? 1 : 0, dtype_, segments ? idx(s_.lay.item_start) : nullptr, seg_items,
                               segments, stream_));
    if (mfma && s_.decode_only) {
      const SplitPlan sp = split_plan(items, nkv * chunks, s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
      float *part_o, *part_ml;
      partials(sp, part_o, part_ml);
      if (leaves_to_product(sp, part_o, part_ml)) out = nullptr;
      ok(me_attention_decode_bf16(q, kc, vc, idx(s_.lay.item_ctx), table, width, out, part_o, part_ml, items, nh, nkv, d, bs, window,
                                  scale, sp.split_keys, sp.num_splits, s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves,
                                  idx(s_.lay.live_items) + 1, stream_));
      return;
    }
    if (mfma) {
      auto it = s_.plans.find({nh, nkv, d, window, 0});
      if (it == s_.plans.end()) throw Error(kBroken, "the step has no work list for a prefill attention layer");
      const StepView::Plan& p = it->second;
      float *part_o = nullptr, *part_ml = nullptr;
      if (p.max_chunks > 1) {
        part_o = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * d * 4);
        part_ml = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * 2 * 4);
      }
      ok(me_attention_prefill_bf16(q, kc, vc, items, table, width, out, idx(p.work), idx(p.bundle_first), p.bundles, part_o, part_ml,
                                   p.token_chunks >= 0 ? idx(p.token_chunks) : nullptr, p.max_chunks, t_, nh, nkv, d, bs, window,
                                   scale, p.columns, stream_));
      return;
    }
    ok(me_attention_general(q, kc, vc, idx(s_.lay.positions), idx(s_.lay.token_item), table, width, out, t_, nh, nkv, d, bs, window,
                            scale, dtype_, items, stream_));
  }

  // Linear attention with a decay per head over the state rows of the step's items.
  void decay_state(const Op& op) {
    const int heads = (int)op.i[0], d = (int)op.i[1], dv = (int)op.i[2], rd = (int)op.i[3];
    const float* rope = (const float*)op.p[1];
    if (rope && op.i[8] < s_.max_ctx)
      throw Error(kBadValue, "the rotary table covers " + std::to_string(op.i[8]) + " positions, the step may reach " +
                                 std::to_string(s_.max_ctx));
    void* ws = arena_.take((size_t)me_decay_state_workspace(t_, s_.lay.items, heads, d, dv));
    int longest = 0;  // (a replayed decode step has no host-side lengths: every item brings one token)
    if (!s_.decode_only && s_.qlens)
      for (int i = 0; i < s_.lay.items; ++i) longest = std::max(longest, s_.qlens[i]);
    ok(me_decay_state(bufs_[op.in], rope, rd, (int)op.i[4], idx(s_.lay.positions), (const float*)op.p[0], (const float*)op.p[2],
                      (float*)op.p[3], idx(s_.lay.item_start), idx(s_.lay.state_slots), bufs_[op.out], ws, t_, s_.lay.items, heads,
                      d, dv, (int)op.i[5], op.f[0], (int)op.i[6], (int)op.i[7], op.f[1], dtype_, longest, stream_));
  }

  // The pending result rewrites the streams (by the coefficients of the part that gave it), the coming part's input is
  // read from them and normed: one kernel.
  void stream_norm(const Op& op, void* out, const int* rows, int num_rows, int write_x) {
    if (!spread_) throw Error(kBroken, "a norm over several streams before the streams begin");
    if (held_.any() || pending_.carried()) throw Error(kBroken, "several streams take one pending result at a time");
    if (pending_.any() && !op.p[op.kind == kOpStreamHead ? 2 : 1])
      throw Error(kBroken, "a result is pending and nothing says how it rewrites the streams");
    if (pending_.any() && pending_.scale != 1.f) throw Error(kBroken, "a result of several streams is not scaled");
    const float* mix_out = pending_.any() ? (const float*)op.p[op.kind == kOpStreamHead ? 2 : 1] : nullptr;
    const float* w_in = op.kind == kOpStreamHead ? nullptr : (const float*)op.p[2];
    ok(me_streams_norm(x_, (long long)t_ * h_, streams_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, mix_out,
                       w_in, (const float*)op.p[0], out, rows, num_rows, h_, op.f[0], write_x, dtype_, stream_));
    pending_ = Pending();
    if (op.kind != kOpStreamHead) release_parts();  // (the head's buffers lie behind waiting partial sums)
  }

  // The rewrite of the streams, the norm and the product behind it: for a row or two of a bfloat16 step all in the
  // product's kernel (every block rewrites and norms the rows while its first weights are on their way; block 0 writes the
  // new streams to the second set of buffers); else the norm as a kernel of its own, then the product.
  void stream_norm_linear(const Op& op) {
    const int rows_of_w = (int)op.i[0], k = (int)op.i[1], gated = (int)op.i[2];
    if (k != h_) throw Error(kBadValue, "a product behind a norm reads the hidden size");
    if (!spread_) throw Error(kBroken, "a norm over several streams before the streams begin");
    if (held_.any() || pending_.carried()) throw Error(kBroken, "several streams take one pending result at a time");
    if (pending_.any() && !op.p[2]) throw Error(kBroken, "a result is pending and nothing says how it rewrites the streams");
    if (pending_.any() && pending_.scale != 1.f) throw Error(kBroken, "a result of several streams is not scaled");
    const int n = gated ? rows_of_w / 2 : rows_of_w;
    const int pending = pending_.parts ? kPendingParts : pending_.delta ? kPendingTensor : kPendingNone;
    if (streams_ <= 4 && choose_norm_fusion(dtype_, t_, rows_of_w, k, pending, compute_units(), true) == kNormInStream) {
      const bool adds = pending_.any();
      ok(me_gemm_bf16_stream_norm_streams(x_, (long long)t_ * h_, streams_, pending_.delta, pending_.parts, pending_.num_parts,
                                          pending_.stride, (const float*)op.p[2], (const float*)op.p[3], (const float*)op.p[0], op.f[0],
                                          adds ? spare_ : nullptr, op.p[1], bufs_[op.out], t_, n, k, gated, dtype_, compute_units(),
                                          stream_));
      if (adds) std::swap(x_, spare_);
      pending_ = Pending();
      release_parts();
      return;
    }
    ok(me_streams_norm(x_, (long long)t_ * h_, streams_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride,
                       pending_.any() ? (const float*)op.p[2] : nullptr, (const float*)op.p[3], (const float*)op.p[0], normed_, nullptr, t_,
                       h_, op.f[0], 1, dtype_, stream_));
    pending_ = Pending();
    release_parts();
    product(normed_, op.p[1], rows_of_w, k, gated, dtype_, bufs_[op.out]);
  }

  void stream_head(const Op& op) {
    const int rows = s_.lay.rows;
    result_.rows = rows;
    if (rows == 0) {
      pending_ = Pending();
      return;
    }
    void* picked = arena_.take((size_t)rows * h_ * elem_);
    stream_norm(op, picked, idx(s_.lay.want_rows), rows, 0);
    logits_of(picked, op);
  }

  // Attention over one cached latent per token (csrc/latent_attention.hip): the latent's norm, the rotation and the page
  // write; the keys' map folded into the queries; attention over one key/value head whose values are the latents; the
  // values' map on the weighted latents, with the output gate.
  void latent_attention(const Op& op) {
    const int nh = (int)op.i[0], d = (int)op.i[1], r = (int)op.i[2], rank = (int)op.i[3], dv = (int)op.i[4], bs = (int)op.i[5];
    const int g = (int)op.i[6], dk = rank + r;
    if (g < 0 || g >= (int)s_.lay.widths.size()) throw Error(kBadValue, "an attention layer names a cache group the step lacks");
    if (op.i[7] < s_.max_ctx)
      throw Error(kBadValue, "the rotary table covers " + std::to_string(op.i[7]) + " positions, the step may reach " +
                                 std::to_string(s_.max_ctx));
    // (the rows may be padded behind the gates, so that every row starts at a multiple of 16 bytes)
    const bool reads_only = op.i[9] != 0;  // another layer's pages: the rows hold no latent projection
    const long long used = (long long)nh * (d + r) + (reads_only ? 0 : dk) + nh, row = values_[op.in].cols;
    if (row < used) throw Error(kBadValue, "the projections of a latent attention layer have the wrong width");
    const int32_t* table = idx(s_.lay.tables[g]);
    const int width = s_.lay.widths[g], items = s_.lay.items;
    const int vr = latent_value_rows(op);  // rows of a value page: the latent's, or the whole key's for the matrix-core kernels
    const float* sink = (const float*)op.p[6];
    const float scale = op.f[1];
    const char* proj = (const char*)bufs_[op.in];
    void* qa = arena_.take((size_t)t_ * nh * dk * elem_);
    void* ol = arena_.take((size_t)t_ * nh * vr * elem_);
    const void *kc = op.p[2], *vc = op.p[3];
    ok(me_latent_prepare_for(proj, row, (const float*)op.p[0], (const float*)op.p[1], idx(s_.lay.positions), idx(s_.lay.token_item), table,
                             width, qa, (void*)kc, (void*)vc, t_, nh, d, r, rank, vr, bs, op.f[0], reads_only ? 0 : 1, dtype_, stream_));
    ok(me_head_product(proj, row, d + r, op.p[4], qa, (long long)nh * dk, dk, nullptr, 0, t_, nh, rank, d, dtype_, stream_));
    if (latent_takes_matrix_cores(op, dtype_) && s_.decode_only) {
      // one new token per item: the split-context kernel; all heads share the one key/value head, 16 to a wave
      if ((long long)width * bs < s_.max_ctx) throw Error(kBadValue, "the block table cannot hold the step's longest context");
      const SplitPlan sp = split_plan(items, (nh + 15) / 16, s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
      float* part_o = (float*)arena_.take((size_t)items * nh * sp.num_splits * dk * 4);
      float* part_ml = (float*)arena_.take((size_t)items * nh * sp.num_splits * 2 * 4);
      // where the launch leaves one partial result per split, one kernel adds them up (with the sink), maps the weighted
      // latents to the heads' values and gates them: no kernel of its own for the sum, none for the values' map
      const bool tail = me_attention_decode_leaves_parts(items, nh, 1, dk, sp.num_splits) && me_latent_values_supported(sp.num_splits, rank);
      ok(me_attention_decode_bf16_sink(qa, kc, vc, idx(s_.lay.item_ctx), table, width, tail ? nullptr : ol, part_o, part_ml, items, nh, 1,
                                       dk, bs, sink, scale, sp.split_keys, sp.num_splits, s_.max_ctx, sp.live, sp.full_splits,
                                       kDecodeWaves, idx(s_.lay.live_items) + 1, stream_));
      if (tail) {
        ok(me_latent_values_bf16(part_o, part_ml, sp.num_splits, dk, rank, sink, op.p[5], proj + (size_t)(used - nh) * elem_, row,
                                 bufs_[op.out], items, nh, dv, stream_));
        return;
      }
    } else if (latent_takes_matrix_cores(op, dtype_)) {
      auto it = s_.plans.find({nh, 1, dk, 0, 0});
      if (it == s_.plans.end()) throw Error(kBroken, "the step has no work list for a latent attention layer");
      const StepView::Plan& p = it->second;
      float *part_o = nullptr, *part_ml = nullptr;
      if (p.max_chunks > 1) {
        part_o = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * dk * 4);
        part_ml = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * 2 * 4);
      }
      ok(me_attention_prefill_bf16_sink(qa, kc, vc, items, table, width, ol, idx(p.work), idx(p.bundle_first), p.bundles, part_o, part_ml,
                                        p.token_chunks >= 0 ? idx(p.token_chunks) : nullptr, p.max_chunks, t_, nh, 1, dk, bs, sink, scale,
                                        p.columns, stream_));
    } else {
      ok(me_attention_general_gated(qa, kc, vc, idx(s_.lay.positions), idx(s_.lay.token_item), table, width, ol, t_, nh, 1, dk, vr, bs,
                                    0, 0, nullptr, 0, scale, sink, nullptr, 0, dtype_, items, stream_));
    }
    ok(me_head_product(ol, (long long)nh * vr, vr, op.p[5], bufs_[op.out], (long long)nh * dv, dv, proj + (size_t)(used - nh) * elem_, row,
                       t_, nh, dv, rank, dtype_, stream_));
  }

  // A feed-forward of routed experts (csrc/routed_ff.hip): its result waits as one partial sum per expert of a token, and one
  // more for an expert that every token uses (two plain products around the activation, which the token's gate multiplies).
  void routed_ff(const Op& op) {
    const int E = (int)op.i[0], top = (int)op.i[1], ff = (int)op.i[2], shared_ff = (int)op.i[7];
    pending_ = Pending();
    pending_.scale = scale_of(op.f[3]);  // what the block multiplies the result by
    parts_mark_ = arena_.used;
    const int sums = top + (shared_ff > 0 ? 1 : 0);
    float* parts = (float*)arena_.take((size_t)sums * t_ * h_ * 4);
    released_to_ = arena_.used;  // the partial sums outlive this operation, its workspace does not
    void* ws = arena_.take((size_t)me_routed_ff_workspace(t_, E, top, ff, elem_));
    float* shared_gate = shared_ff > 0 && !op.i[9] ? (float*)arena_.take((size_t)t_ * 4) : nullptr;
    ok(me_routed_ff_routed(bufs_[op.in], (const float*)op.p[0], op.p[1], op.p[2], parts, ws, t_, h_, E, top, ff, (int)op.i[3], op.f[0],
                           (int)op.i[4], (int)std::max<int64_t>(op.i[5], 1), (int)std::max<int64_t>(op.i[6], 1), scale_of(op.f[1]),
                           shared_gate, (int)op.i[8], (const float*)op.p[5], dtype_, stream_));
    if (shared_ff > 0 && act_code_is_ungated((int)op.i[3])) {  // an expert without a gate: up, the activation, down
      void* up = arena_.take((size_t)t_ * shared_ff * elem_);
      product(bufs_[op.in], op.p[3], shared_ff, h_, 0, dtype_, up);
      if (shared_gate) throw Error(kBadValue, "a shared expert without gate rows has no gate of its own either");
      ok(me_act_rows(up, up, (long long)t_ * shared_ff, (int)op.i[3], dtype_, stream_));
      product(up, op.p[4], h_, shared_ff, 0, kF32, parts + (size_t)top * t_ * h_);
    } else if (shared_ff > 0) {
      void* gu = arena_.take((size_t)t_ * 2 * shared_ff * elem_);
      void* act = arena_.take((size_t)t_ * shared_ff * elem_);
      product(bufs_[op.in], op.p[3], 2 * shared_ff, h_, 0, dtype_, gu);
      ok(me_gated_rows(gu, shared_gate, act, t_, shared_ff, (int)op.i[3], op.f[2], dtype_, stream_));
      product(act, op.p[4], h_, shared_ff, 0, kF32, parts + (size_t)top * t_ * h_);
    }
    pending_.parts = parts;
    pending_.num_parts = sums;
    pending_.stride = (long long)t_ * h_;
  }

  // Attention over a sliding window and the means of whole blocks of keys before it (csrc/pooled_attention.hip, then the general
  // attention kernel with the pooled entries as a run of their own).
  void pooled_attention(const Op& op) {
    const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2], dv = (int)op.i[3], bs = (int)op.i[4];
    const int window = (int)op.i[5], pool = (int)op.i[6], g = (int)op.i[7];
    if (g < 0 || g >= (int)s_.lay.widths.size()) throw Error(kBadValue, "an attention layer names a cache group the step lacks");
    const int32_t* table = idx(s_.lay.tables[g]);
    const int width = s_.lay.widths[g];
    const long long row = values_[op.in].cols, out_row = values_[op.out].cols;
    void* q = arena_.take((size_t)t_ * nh * d * elem_);
    const int rotary = (int)op.i[12], taps = (int)op.i[14];
    const float* sink = (const float*)op.p[9];
    const float softcap = op.f[3];
    if (rotary > 0 && op.i[13] < s_.max_ctx)
      throw Error(kBadValue, "the rotary table covers " + std::to_string(op.i[13]) + " positions, the step may reach " + std::to_string(s_.max_ctx));
    if (rotary > 0 || taps > 0) {
      if (pool > 0 || op.i[10] < 0) throw Error(kBadValue, "a convolution or a rotation ahead of attention with pooled blocks or without a value projection");
      ok(me_conv_norm_rope_scatter(bufs_[op.in], row, (int)op.i[8], (int)op.i[9], (int)op.i[10], (const float*)op.p[7], taps, (float*)op.p[8],
                                   idx(s_.lay.state_slots), idx(s_.lay.item_start), (const float*)op.p[0], (const float*)op.p[1],
                                   (const float*)op.p[6], rotary, idx(s_.lay.positions), idx(s_.lay.token_item), table, width, q, (void*)op.p[2],
                                   (void*)op.p[3], t_, s_.lay.items, nh, nkv, d, dv, bs, op.f[0], dtype_, stream_));
    } else
    ok(me_whole_norm_scatter_step(bufs_[op.in], row, (int)op.i[8], (int)op.i[9], (int)op.i[10], (const float*)op.p[0],
                                  (const float*)op.p[1], idx(s_.lay.positions), idx(s_.lay.token_item), table, width, q, (void*)op.p[2],
                                  (void*)op.p[3], (void*)op.p[4], (void*)op.p[5], t_, nh, nkv, d, dv, bs, pool, op.f[0],
                                  s_.decode_only ? 1 : 0, dtype_, stream_));
    const float out_scale = op.f[2];  // (always given; nought is a scale like any other)
    if (pooled_takes_matrix_cores(op, dtype_, out_row) && s_.decode_only) {
      // one new token per item: the split-context kernel, which deals the pooled entries' tiles to its splits before the window's
      const int items = s_.lay.items;
      if ((long long)width * bs < s_.max_ctx) throw Error(kBadValue, "the block table cannot hold the step's longest context");
      const SplitPlan sp = split_plan(items, nkv * ((nh / nkv + 15) / 16), s_.max_ctx, s_.least_live, idx(s_.lay.live_items));
      float* part_o = (float*)arena_.take((size_t)items * nh * sp.num_splits * d * 4);
      float* part_ml = (float*)arena_.take((size_t)items * nh * sp.num_splits * 2 * 4);
      if (pool > 0)
        ok(me_attention_decode_bf16_pooled(q, op.p[2], op.p[3], op.p[4], op.p[5], pool, idx(s_.lay.item_ctx), table, width, bufs_[op.out],
                                           out_row, (int)op.i[11], out_scale, part_o, part_ml, items, nh, nkv, d, bs, window, op.f[1],
                                           sp.split_keys, sp.num_splits, s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves,
                                           idx(s_.lay.live_items) + 1, stream_));
      else
        ok(me_attention_decode_bf16_placed(q, op.p[2], op.p[3], idx(s_.lay.item_ctx), table, width, bufs_[op.out], out_row, (int)op.i[11],
                                           out_scale, part_o, part_ml, items, nh, nkv, d, bs, window, op.f[1], softcap, sink, sp.split_keys,
                                           sp.num_splits, s_.max_ctx, sp.live, sp.full_splits, kDecodeWaves, idx(s_.lay.live_items) + 1,
                                           stream_));
      return;
    }
    if (pooled_takes_matrix_cores(op, dtype_, out_row)) {
      // prompts and portions: the tiled kernel, whose work list has an entry of its own for a tile's pooled entries
      auto it = s_.plans.find({nh, nkv, d, window, 0, pool});
      if (it == s_.plans.end()) throw Error(kBroken, "the step has no work list for an attention layer with pooled blocks");
      const StepView::Plan& p = it->second;
      float *part_o = nullptr, *part_ml = nullptr;
      if (p.max_chunks > 1) {
        part_o = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * d * 4);
        part_ml = (float*)arena_.take((size_t)t_ * nh * p.max_chunks * 2 * 4);
      }
      if (pool > 0)
        ok(me_attention_prefill_bf16_pooled(q, op.p[2], op.p[3], op.p[4], op.p[5], pool, s_.lay.items, table, width, bufs_[op.out], out_row,
                                            (int)op.i[11], out_scale, idx(p.work), idx(p.bundle_first), p.bundles, part_o, part_ml,
                                            p.token_chunks >= 0 ? idx(p.token_chunks) : nullptr, p.max_chunks, t_, nh, nkv, d, bs, window,
                                            op.f[1], p.columns, stream_));
      else
        ok(me_attention_prefill_bf16_placed(q, op.p[2], op.p[3], s_.lay.items, table, width, bufs_[op.out], out_row, (int)op.i[11], out_scale,
                                            idx(p.work), idx(p.bundle_first), p.bundles, part_o, part_ml,
                                            p.token_chunks >= 0 ? idx(p.token_chunks) : nullptr, p.max_chunks, t_, nh, nkv, d, bs, window,
                                            op.f[1], softcap, sink, p.columns, stream_));
      return;
    }
    ok(me_attention_general_capped(q, op.p[2], op.p[3], idx(s_.lay.positions), idx(s_.lay.token_item), table, width, bufs_[op.out], t_, nh,
                                   nkv, d, dv, bs, window, 0, nullptr, 0, op.f[1], sink, nullptr, 0, op.p[4], op.p[5], pool, out_row,
                                   (int)op.i[11], out_scale, softcap, dtype_, s_.lay.items, stream_));
  }

  // Linear attention by the generalized delta rule over the state rows of the step's items (csrc/delta_rule.hip).
  void delta_rule(const Op& op) {
    const int heads = (int)op.i[0], d = (int)op.i[1];
    if (t_ > s_.lay.items) {
      // an item brings more than one token: the walk over the tokens does nothing but the recurrence (what every token can
      // have ahead of it, and what it is owed afterwards, runs for all tokens at once)
      void* ws = arena_.take((size_t)me_delta_rule_workspace(t_, heads, d));
      ok(me_delta_rule_steps(bufs_[op.in], values_[op.in].cols, (int)op.i[3], (int)op.i[4], (int)op.i[5], (int)op.i[6], (int)op.i[7],
                             (int)op.i[8], op.p[0], (const float*)op.p[1], (const float*)op.p[2], (const float*)op.p[3], (float*)op.p[4],
                             idx(s_.lay.item_start), idx(s_.lay.state_slots), bufs_[op.out], values_[op.out].cols, (int)op.i[9], op.f[2],
                             t_, s_.lay.items, heads, d, (int)op.i[2], op.f[0], op.f[1], dtype_, ws, stream_));
      return;
    }
    ok(me_delta_rule(bufs_[op.in], values_[op.in].cols, (int)op.i[3], (int)op.i[4], (int)op.i[5], (int)op.i[6], (int)op.i[7], (int)op.i[8],
                     op.p[0], (const float*)op.p[1], (const float*)op.p[2], (const float*)op.p[3], (float*)op.p[4],
                     idx(s_.lay.item_start), idx(s_.lay.state_slots), bufs_[op.out], values_[op.out].cols, (int)op.i[9],
                     op.f[2], t_, s_.lay.items, heads, d, (int)op.i[2], op.f[0], op.f[1], dtype_, stream_));
  }

  // Rows are selected before the final norm, as the reference does (model.py:186); logits are float32.
  void head(const Op& op) {
    const int rows = s_.lay.rows;
    result_.rows = rows;
    if (rows == 0) {
      pending_ = held_ = Pending();
      return;
    }
    void* picked = arena_.take((size_t)rows * h_ * elem_);
    if (held_.any() && held_.scale != pending_.scale && pending_.any()) add_held();
    if (groups_of(op.i[0]) > 1 || pending_.scale != 1.f || held_.any()) {
      const float scale = pending_.any() ? pending_.scale : held_.scale;
      ok(me_add_group_rmsnorm2(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, held_.delta, held_.parts,
                               held_.num_parts, held_.stride, scale, (const float*)op.p[0], picked, idx(s_.lay.want_rows), rows, h_,
                               groups_of(op.i[0]), op.f[0], 0, dtype_, stream_));
      held_ = Pending();
    } else
      ok(me_add_rmsnorm(x_, pending_.delta, pending_.parts, pending_.num_parts, pending_.stride, (const float*)op.p[0], picked,
                        idx(s_.lay.want_rows), rows, h_, op.f[0], 0, dtype_, stream_));
    pending_ = Pending();
    logits_of(picked, op);
  }

  // The head behind a final norm that a part computed itself: the value's first rows are the normed wanted rows.
  void head_rows(const Op& op) {
    result_.rows = s_.lay.rows;
    if (s_.lay.rows == 0) return;
    logits_of(bufs_[op.in], op);
  }

  void logits_of(const void* picked, const Op& op) {
    const int rows = s_.lay.rows, vocab = prog_.vocab();
    float* logits = (float*)arena_.take((size_t)rows * vocab * 4);
    product(picked, op.p[1], vocab, h_, 0, kF32, logits, kRoleHead, rows);
    if (op.f[1] != 1.f) ok(me_scale_f32(logits, op.f[1], (long long)rows * vocab, stream_));
    result_.logits = logits;
  }

  // A part that brings its own code: it reads and writes values of the step and launches on the step's stream.
  void call(const Op& op) {
    CallFrame f{};
    f.context = (void*)op.p[1];
    f.in = op.in >= 0 ? bufs_[op.in] : nullptr;
    f.out = op.out >= 0 ? bufs_[op.out] : nullptr;
    f.x = x_;
    f.in_cols = op.in >= 0 ? values_[op.in].cols : 0;
    f.out_cols = op.out >= 0 ? values_[op.out].cols : 0;
    f.in_elem = op.in >= 0 ? values_[op.in].elem : 0;
    f.out_elem = op.out >= 0 ? values_[op.out].elem : 0;
    f.tokens = t_;
    f.rows = s_.lay.rows;
    f.stream = stream_;
    if (!op.p[0]) throw Error(kBadValue, "a called part needs its function");
    if (((CallFn)op.p[0])(&f) != 0) throw Error(kBadState, "a part's own code failed in a step");
  }

  void sample() {
    const int rows = s_.lay.rows;
    if (rows == 0 || !result_.logits) return;
    int32_t* drawn = fed_tokens_ ? fed_tokens_ : (int32_t*)arena_.take((size_t)rows * 4);
    void* ws = arena_.take((size_t)rows * me_sample_chunks(prog_.vocab()) * 8);
    ok(me_sample(result_.logits, rows, prog_.vocab(), (const float*)idx(s_.lay.temperatures),
                 (const uint64_t*)idx(s_.lay.sample_keys), drawn, ws, stream_));
    result_.drawn = drawn;
  }

  const Program& prog_;
  const std::vector<Value>& values_;
  const StepView& s_;
  Arena& arena_;
  int32_t* fed_tokens_;
  hipStream_t stream_;
  const int dtype_, elem_, t_, h_, streams_;
  bool spread_ = false;  // the streams are in use (kOpStreams has run)
  float *x_, *spare_;
  void* normed_;
  std::vector<void*> bufs_;
  Pending pending_, held_;  // held_: a result set aside (kOpHold) until the add that takes it together with pending_
  size_t held_mark_ = (size_t)-1;
  struct AttnParts {  // what a decode attention left for the output projection behind it
    float *o = nullptr, *ml = nullptr;
    int splits = 0, nh = 0, d = 0, value = -1;
    size_t mark = 0;
  } attn_parts_;
  const Op* next_ = nullptr;  // the operation behind the one being run
  size_t parts_mark_ = (size_t)-1, released_to_ = (size_t)-1;
  RunResult result_;
};

}  // namespace

RunResult Program::run(const StepView& s, char* arena, size_t arena_bytes, int32_t* fed_tokens, hipStream_t stream) const {
  Arena a{arena, arena_bytes};
  Run run(*this, values_, s, a, fed_tokens, stream);
  return run.go();
}

std::vector<std::vector<int>> Program::prefill_geometries() const {
  std::vector<std::vector<int>> out;
  if (dtype_ != kBF16) return out;
  for (const Op& op : ops_) {
    if (op.kind == kOpLatentAttention && latent_takes_matrix_cores(op, dtype_)) {
      std::vector<int> key = {(int)op.i[0], 1, (int)(op.i[3] + op.i[2]), 0, 0};
      if (std::find(out.begin(), out.end(), key) == out.end()) out.push_back(key);
    }
    if (op.kind == kOpPooledAttention && pooled_takes_matrix_cores(op, dtype_, values_[op.out].cols)) {
      std::vector<int> key = {(int)op.i[0], (int)op.i[1], (int)op.i[2], (int)op.i[5], 0, (int)op.i[6]};
      if (std::find(out.begin(), out.end(), key) == out.end()) out.push_back(key);
    }
    if (op.kind != kOpAttention) continue;
    const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2], bs = (int)op.i[4], window = (int)op.i[5];
    if (!attention_is_plain(op) && !attention_takes_tiled_prefill(op, dtype_)) continue;
    if (!me_attention_mfma_supported(d, bs) || nh / nkv > 16) continue;
    std::vector<int> key = {nh, nkv, d, window, attention_is_plain(op) ? 0 : (int)op.i[10]};
    if (std::find(out.begin(), out.end(), key) == out.end()) out.push_back(key);
  }
  return out;
}

size_t Program::arena_need(int64_t tokens, int64_t items, int64_t rows, int64_t max_ctx) const {
  const size_t elem = dtype_ == kF32 ? 4 : 2;
  const size_t pad = 256;
  size_t fixed = 2 * (size_t)streams_of(ops_) * ((size_t)tokens * hidden_ * 4 + pad) + (size_t)tokens * hidden_ * elem + pad;
  for (const Value& v : values_) fixed += (size_t)tokens * v.cols * v.elem + pad;
  size_t scratch = 0;
  for (const Op& op : ops_) {
    size_t need = 0;
    if (op.kind == kOpNormLinear || op.kind == kOpLinear || op.kind == kOpStreamNormLinear) need = (size_t)tokens * op.i[0] * 4 + pad;
    if (op.kind == kOpLinearDelta)  // up to 16 partial sums of up to 64 rows, or one float32 result of all rows
      need = std::max<size_t>((size_t)kMaxRuns * std::min<int64_t>(tokens, kSmallMaxRows), (size_t)tokens) * op.i[0] * 4 + pad;
    if (op.kind == kOpDecayState)
      need = (size_t)me_decay_state_workspace(tokens, items, (int)op.i[0], (int)op.i[1], (int)op.i[2]) + pad;
    if (op.kind == kOpLatentAttention) {
      const int nh = (int)op.i[0], dk = (int)(op.i[3] + op.i[2]);
      need = (size_t)tokens * nh * 2 * dk * elem + 2 * pad;
      if (latent_takes_matrix_cores(op, dtype_)) {  // the splits' partial results of a decode step, or those of cut tiles
        size_t most = 0;
        for (int64_t b = 1; b <= items; ++b) {
          int keys, splits;
          decode_splits((int)std::max<int64_t>(1, (b + 1) / 2), (nh + 15) / 16, (int)max_ctx, keys, splits);
          most = std::max(most, (size_t)b * splits);
        }
        const size_t decode = most * nh * (dk + 2) * 4 + 2 * pad;
        const size_t prefill = (size_t)(256ll << 20) + (size_t)(256ll << 20) * 2 / dk + (size_t)tokens * nh * 8 + 2 * pad;
        need += std::max(decode, tokens > items ? prefill : (size_t)0);
      }
    }
    if (op.kind == kOpRoutedFF)
      need = (size_t)(op.i[1] + 1) * tokens * hidden_ * 4 + (size_t)me_routed_ff_workspace(tokens, (int)op.i[0], (int)op.i[1], (int)op.i[2], (int)elem) +
             (size_t)tokens * (4 + 3 * op.i[7] * elem + 2 * op.i[7] * 4) + 6 * pad;
    if (op.kind == kOpTimeMix)
      need = (size_t)tokens * (5 * hidden_ + 4 * op.i[0] * op.i[1] + op.i[2]) * elem + (size_t)me_time_mix_workspace(tokens, (int)op.i[0], (int)op.i[1]) +
             (size_t)std::min<int64_t>(tokens, kTimeMixStackedTokens) * 5 * (hidden_ + 4 * op.i[0] * op.i[1] + op.i[2]) * elem + 16 * pad;
    if (op.kind == kOpDeltaRule && tokens > items) need = (size_t)me_delta_rule_workspace(tokens, (int)op.i[0], (int)op.i[1]) + pad;
    if (op.kind == kOpPooledAttention) {
      need = (size_t)tokens * op.i[0] * op.i[2] * elem + pad;
      if (dtype_ == kBF16 && op.i[3] == op.i[2] && me_attention_mfma_supported((int)op.i[2], (int)op.i[4]) && op.i[0] / op.i[1] <= 16) {
        const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2];
        size_t most = 0;  // the splits' partial results of a decode step
        for (int64_t b = 1; b <= items; ++b) {
          int keys, splits;
          decode_splits((int)std::max<int64_t>(1, (b + 1) / 2), nkv * ((nh / nkv + 15) / 16), (int)max_ctx, keys, splits);
          most = std::max(most, (size_t)b * splits);
        }
        const size_t decode = most * nh * (d + 2) * 4 + 2 * pad;
        // partial results of cut tiles: the work list's bound, and one chunk more for the pooled entries
        const size_t prefill = (size_t)(256ll << 20) + (size_t)(256ll << 20) * 2 / d + (size_t)tokens * nh * (d + 2) * 4 * 2 + 2 * pad;
        need += std::max(decode, tokens > items ? prefill : (size_t)0);
      }
    }
    if (op.kind == kOpAttention && !attention_is_plain(op)) {
      need = (size_t)tokens * op.i[0] * op.i[2] * elem + pad;
      if (attention_takes_tiled_prefill(op, dtype_)) {  // the splits' partial results of a decode step
        const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2];
        size_t most = 0;
        for (int64_t b = 1; b <= items; ++b) {
          int keys, splits;
          decode_splits((int)std::max<int64_t>(1, (b + 1) / 2), nkv * ((nh / nkv + 15) / 16), (int)max_ctx, keys, splits);
          most = std::max(most, (size_t)b * splits);
        }
        need += most * nh * (d + 2) * 4 + 2 * pad;
      }
      if (attention_takes_tiled_prefill(op, dtype_) && tokens > items)  // partial results of cut tiles: the work list's bound,
        need += (size_t)(256ll << 20) + (size_t)(256ll << 20) * 2 / op.i[2] +  // and one chunk more for the kept first keys
                (size_t)tokens * op.i[0] * (op.i[2] + 2) * 4 * 2 + 2 * pad;
    } else if (op.kind == kOpAttention) {
      const int nh = (int)op.i[0], nkv = (int)op.i[1], d = (int)op.i[2];
      const int chunks = (nh / nkv + 15) / 16;
      size_t most = 0;  // items x splits at its largest over the batch sizes a launch may hold
      for (int64_t b = 1; b <= items; ++b) {
        int keys, splits;
        decode_splits((int)std::max<int64_t>(1, (b + 1) / 2), nkv * chunks, (int)max_ctx, keys, splits);
        most = std::max(most, (size_t)b * splits);
      }
      const size_t decode = most * nh * (d + 2) * 4 + 2 * pad;
      const size_t prefill = (size_t)(256ll << 20) + (size_t)(256ll << 20) * 2 / d + (size_t)tokens * nh * 8 + 2 * pad;
      need = (size_t)tokens * nh * d * elem + pad + std::max(decode, tokens > items ? prefill : (size_t)0);
    }
    scratch = std::max(scratch, need);
  }
  const size_t tail = (size_t)rows * hidden_ * elem + (size_t)rows * vocab_ * 4 + (size_t)rows * 4 +
                      (size_t)rows * me_sample_chunks(vocab_) * 8 + 4 * pad;
  // partial sums of the last delta wait beside the head's buffers
  return fixed + 2 * scratch + tail + std::max<size_t>((size_t)kMaxRuns * kSmallMaxRows, (size_t)tokens) * hidden_ * 4 + (1 << 16);
}

}  // namespace me

// A plain bfloat16 product through the GEMM library, with this folder's kernels where the library has no algorithm:
// what the step program calls for a product that choose_product leaves to the library, for callers outside it.
extern "C" int me_gemm_bf16_any(const void* x, const void* w, void* out, int m, int n, int k, int out_dtype, hipStream_t stream) {
  try {
    me::library_product(x, w, out, m, n, k, out_dtype, stream);
    return 0;
  } catch (const std::exception& e) {
    return me_fail("%s", e.what());
  }
}
