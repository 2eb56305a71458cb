// The native step program: a model's forward pass as a list of operations that C++ runs from one
// call, so that a step costs the host one call, not one per kernel. The Python parts write their
// operations into it once, when the model is built (each part knows what it computes, none knows the
// model it is in); which kernel serves an operation is decided per step from the step's size.
//
// State that the operations share: the residual stream x (float32 [tokens, hidden]) in one of two
// buffers, and a pending delta (a part's output that the next norm adds to x while it norms): nothing,
// a buffer in the compute dtype, partial sums over runs of k that the add sums up, or, where the delta's
// product has added itself to x already, the first half of the norm behind it (the rows times the norm's
// weight, and their sums of squares) for the product after the norm to finish.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <map>
#include <string>
#include <vector>

#include "core.h"
#include "prefill_plan.h"

namespace me {

enum OpKind {
  kOpEmbed = 0,       // p0 table, f0 the multiplier on the looked-up rows; -> x
  kOpNormLinear = 1,  // p0 norm weight, f0 eps, p1 W [rows, K], i0 rows of W, i1 K, i2 gated, i3 groups of the norm (0: one);
                      // pending + x -> out
  kOpNorm = 2,        // p0 norm weight, f0 eps, i0 groups of the norm (0: one); pending + x -> out [tokens, hidden]. i1 != 0: a second
                      // norm of the same stream (nothing is pending; a result that was set aside stays aside)
  kOpLinear = 3,      // in, p1 W, i0 rows of W, i1 K, i2 gated -> out
  kOpLinearDelta = 4, // in, p1 W, i0 rows of W (= hidden), i1 K, f0 what the block multiplies the delta by (0: 1) -> pending
  kOpDelta = 5,       // in, f0 what the block multiplies the delta by (0: 1) -> pending
  kOpAttention = 6,   // in qkv, p0 q-norm weight, p1 k-norm weight, p2 rotary table, p3 key pages, p4 value pages;
                      // i0 heads, i1 kv heads, i2 head size, i3 rotary size, i4 page size, i5 window, i6 writes pages,
                      // i7 cache group, i8 positions the table covers; f0 eps, f1 scale -> out [tokens, heads * value size].
                      // Beyond the plain form: i9 size of the value heads (0: the head size), i10 first keys that stay visible
                      // behind the window, i11 pairing of the rotation (0: j with j + r/2; 1: 2j with 2j + 1), i12 values are
                      // turned by their position and outputs turned back (0: no; 1 + the pairing), p5 the table of those angles
  kOpHead = 7,        // p0 final norm weight, f0 eps, p1 head W [vocab, hidden], f1 the scale on the logits, i0 groups of the
                      // norm (0: one) -> logits of the wanted rows
  kOpSample = 8,      // logits -> one token per wanted row
  kOpAdd = 9,         // pending + x -> x, as a kernel of its own (before a norm that is no RMS norm)
  kOpCall = 10,       // a part that brings its own code: p0 a function `int (const CallFrame*)`, p1 its context;
                      // in (or -1), out (or -1): the values it reads and writes. It launches on the step's stream.
  kOpHeadRows = 11,   // in: a value whose first rows are the normed wanted rows; p1 head W, f1 the scale on the logits
  kOpDecayState = 12, // in: projections [tokens, heads (d | d | dv | dv)] (q, k, v, gate); p0 decay float32 [2, heads],
                      // p1 rotary table, p2 weight of the norm over all heads, p3 the state rows [slots, heads, d, dv];
                      // i0 heads, i1 d, i2 dv, i3 rotary size, i4 pairing, i5 activation of q, k, v, i6 kind of the output norm,
                      // i7 activation of the gate, i8 positions the table covers; f0 scale on k, f1 eps
                      // -> out [tokens, heads * dv]
  kOpHold = 13,       // the pending delta is set aside until the next add: a second part that reads the same normed input
                      // follows, and the add takes both results at once (with the same multiplier)
  kOpStreams = 14,    // i0 S: from here on a token has S residual streams [S, tokens, hidden], each a copy of x as it is now
  kOpStreamNorm = 15, // p0 norm weight, f0 eps, p1 float32 [S * S + S]: how the pending result rewrites the streams (mix[from, to],
                      // then out[to]; null: nothing is pending), p2 float32 [S]: what the coming part reads of each stream;
                      // pending + streams -> streams, out [tokens, hidden]
  kOpStreamHead = 16, // p0 final norm weight, f0 eps, p1 head W, f1 the scale on the logits, p2 as p1 of kOpStreamNorm: the sum of the
                      // streams of the wanted rows, normed -> logits
  kOpLatentAttention = 17,  // in: projections [tokens, heads (d + r) | rank + r | heads] (queries, the latent and the shared rotated
                      // key part, a gate per head); p0 weight of the latent's norm, p1 rotary table [positions, 2, r/2], p2 key
                      // pages [page, 1, slot, rank + r], p3 value pages [page, 1, rank, slot], p4 the keys' map per head, transposed
                      // [heads, rank, d], p5 the values' map per head [heads, dv, rank], p6 sink float32 [heads] or null;
                      // i0 heads, i1 d, i2 r, i3 rank, i4 dv, i5 page size, i6 cache group, i7 positions the table covers,
                      // i8 rows of a value page (0: rank; rank + r: the whole key, as the matrix-core kernels want it);
                      // f0 eps, f1 scale -> out [tokens, heads * dv]
  kOpRoutedFF = 18,   // in: normed activations; p0 router W float32 [E, hidden], p1 experts' gate and up rows [E, 2 ff, hidden],
                      // p2 experts' down rows [E, hidden, ff]; i0 E, i1 experts a token, i2 ff, i3 code of the activation
                      // -> pending (partial sums, one per expert of a token). f0 the activation's limit; i4 how the picks are scored
                      // (0: softmax over the picked logits; 1: sigmoid scores over their sum, times f1, picks bounded to the i6 best of
                      // i5 groups). i7 > 0: an expert of that size that every token uses, p3 its gate and up rows [2 i7, hidden], p4
                      // its down rows [hidden, i7], f2 its limit; the router then has one more row, whose sigmoid multiplies it. f3 what the block
                      // multiplies the result by (0: 1)
  kOpStreamNormLinear = 19,  // kOpStreamNorm and the product behind it: p0 norm weight, f0 eps, p1 W [rows, hidden], p2 how the pending
                      // result rewrites the streams (or null), p3 what the product's part reads of each stream; i0 rows of W, i1 K,
                      // i2 gated; pending + streams -> streams, out
  kOpPooledAttention = 20,  // attention over a window and the means of whole blocks of keys before it. in: projections, queries at column
                      // i8 (heads * d), keys at i9 (kv heads * d), values at i10 (kv heads * dv; -1: the values are the keys as projected);
                      // p0, p1 float32 weights of the norms over the whole of q and of k, p2 key pages, p3 value pages, p4, p5 the pooled
                      // blocks' pages; i0 heads, i1 kv heads, i2 d, i3 dv, i4 page size, i5 window, i6 keys a pooled block, i7 cache group;
                      // f0 eps, f1 scale, f2 what multiplies the result -> out, at column i11 (heads * dv wide)
  kOpDeltaRule = 21,  // linear attention by the generalized delta rule. in: projections, the columns i3 r, i4 k, i5 v, i6 gate, i7 a
                      // (heads * d each), i8 the decay's inner projection (i2 wide); p0 the decay's outer weight [heads * d, i2], p1 its
                      // bias, p2 the bias of a, p3 weight of the output norm (float32 [heads * d] each), p4 state rows [slots, heads, d, d];
                      // i0 heads, i1 d; f0 eps, f1 the decay's coefficient, f2 what multiplies the result -> out, at column i9
  kOpResultNorm = 22, // a block that norms a sublayer's result, not its input: x += scale * rmsnorm(pending) * p0 (f0 eps; the scale is the
                      // pending result's), then out (or -1) = x in the compute dtype, which the next sublayer reads. Nothing pending
                      // (p0 may be null): only x -> out
  kOpTokenGate = 23,  // in z [tokens, n]; p0 a table [vocab, i1] in the compute dtype; out [tokens, n] = act(z) * table[token, i0 .. i0 + n - 1],
                      // i2 the activation's code (MeAct)
  kOpActivate = 24,   // in -> out (the same value or another of its size): act(in) elementwise, i0 the activation's code (MeAct)
  kOpTimeMix = 25,    // linear attention with a decay per token and channel and a bonus for the current token (csrc/time_mix.hip). in: the
                      // sublayer's input [tokens, hidden]; p0 float32 [5, hidden] the blends' mu (r, k, v, gate, decay), p1, p8, p9, p10 W_r, W_k, W_v, W_gate
                      // [n, hidden] each (p11, or null: the five weights stacked, [4 n + i2, hidden], for steps of few tokens), p2 W1 [i2, hidden], p3 W2 [n, i2], p4 w0, p5 bonus, p6 weight of the output norm (float32 [n]
                      // each), p7 state rows float32 [slots, i4]: S [heads, d, d], then at i5 the input of the sequence's last token;
                      // i0 heads, i1 d (n = i0 * i1), i2 the decay's inner size, i3 the result's column in out; f0 eps, f1 what multiplies the result
};
// kOpPooledAttention beyond i11: p6 a rotary table [positions, 2, i12 / 2] (i13 positions) that q and k are turned by behind their norm
// (pairs of halves), i12 the turned elements of a head; i14 taps of a short causal convolution over time on every channel of q, k and
// v ahead of the norm, p7 its weights float32 [nq + nk + nv, taps], p8 its state rows float32 [slots, (taps - 1) (nq + nk + nv)];
// p9 float32 [heads] logits that count once in the softmax's denominator and have no value (null: none); f3 > 0: scores are bounded,
// f3 * tanh(score / f3).
// kOpLatentAttention i9 != 0: the layer reads another layer's pages; its rows hold no latent projection ([heads (d + r) | heads]).
// kOpRoutedFF i8: identity experts (router outputs behind the experts' that stand for the token's input itself), p5 float32 correction
// added to the scores for the choice alone (scoring 2: softmax over all outputs); i9 != 0: the shared expert has no gate of its own.
// An activation code of MeAct (16 and more): the experts have no gate rows, p1 is [E, ff, hidden], p3 [i7, hidden].
// kOpLinearDelta i2: the result stays pending whatever the step's size (no product adds itself to the stream).
// kOpAttention beyond i12: i13 every (0: none) and f2 coef of a temperature on the queries, 1 + coef * ln(floor((position + 1) / every)
// + 1); i14: the input ends in one more column per head, a gate whose sigmoid multiplies the head's output.

constexpr int kOpPtrs = 12;

constexpr int kOpInts = 16, kOpFloats = 4;

// What a called part is handed (kOpCall). Pointers are device memory of this step: they change from step to step.
struct CallFrame {
  void* context;
  const void* in;   // [tokens, in_cols] or null
  void* out;        // [tokens, out_cols] or null
  float* x;         // the residual stream, float32 [tokens, hidden]
  int64_t in_cols, out_cols;
  int32_t in_elem, out_elem;  // bytes per element
  int32_t tokens, rows;
  hipStream_t stream;
};
typedef int (*CallFn)(const CallFrame*);

struct Op {
  int kind = 0, in = -1, out = -1;
  const void* p[kOpPtrs] = {nullptr};
  int64_t i[kOpInts] = {0};
  float f[kOpFloats] = {0.f, 0.f, 0.f, 0.f};
};

struct Value {
  int64_t cols;
  int elem;  // bytes per element
};

// What a run needs to know of its step.
struct StepView {
  const int32_t* dev = nullptr;  // the packed index buffer on the device
  StepLayout lay;
  const int* starts = nullptr;  // host: first position and token count of every item
  const int* qlens = nullptr;
  int max_ctx = 1;
  bool decode_only = true;
  int least_live = 0;  // the fewest live items a replay of this launch will hold (= items for an eager step)
  bool fed = false;  // token ids may come from the tokens the step before drew (the token_source section says which)
  // prefill plans behind the indices, by attention geometry (heads, kv heads, head size, window)
  struct Plan {
    int work = 0, bundle_first = 0, token_chunks = -1, bundles = 0, max_chunks = 1, columns = 0;
  };
  std::map<std::vector<int>, Plan> plans;
};

struct RunResult {
  float* logits = nullptr;
  int32_t* drawn = nullptr;
  int rows = 0;
};

class Program {
 public:
  Program(int dtype, int hidden, int vocab) : dtype_(dtype), hidden_(hidden), vocab_(vocab) {}
  int add_value(int64_t cols, int elem) {
    values_.push_back({cols, elem});
    return (int)values_.size() - 1;
  }
  void add_op(const Op& op) { ops_.push_back(op); }
  int dtype() const { return dtype_; }
  int hidden() const { return hidden_; }
  int vocab() const { return vocab_; }
  const std::vector<Op>& ops() const { return ops_; }
  // Bytes of arena that a step of these sizes may need.
  size_t arena_need(int64_t tokens, int64_t items, int64_t rows, int64_t max_ctx) const;
  RunResult run(const StepView& s, char* arena, size_t arena_bytes, int32_t* fed_tokens, hipStream_t stream) const;
  // Distinct attention geometries that take the matrix-core prefill kernel (their steps need a work list).
  std::vector<std::vector<int>> prefill_geometries() const;

 private:
  int dtype_, hidden_, vocab_;
  std::vector<Value> values_;
  std::vector<Op> ops_;
};

}  // namespace me
