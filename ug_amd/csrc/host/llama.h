// ug-llama: the model graph (ug-llama/src/model.rs) over any ug::Device, plus the five custom
// ops a device has to bring (`trait Device` of ug-llama/src/main.rs:22-28).
#pragma once
#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "ug/lazy_buffer.h"

namespace ug_llama {

using LB = ug::LazyBuffer;

// ug-llama/src/main.rs:22-28
struct Ops {
  virtual ~Ops() = default;
  virtual LB rope_i(const LB& src, const LB& cos, const LB& sin, const LB& pos) const = 0;
  virtual LB rope(const LB& src, const LB& cos, const LB& sin, const LB& pos) const = 0;
  virtual LB cat(const LB& lhs, const LB& rhs, size_t axis) const = 0;
  virtual LB custom_softmax(const LB& src) const = 0;
  virtual LB causal_mask(const LB& src) const = 0;

  // Optional fusions (not part of the reference's trait).  The defaults compose the ops above
  // exactly as ug-llama/src/model.rs:231-244 does; a device may answer with one kernel.
  // softmax(causal_mask(att)) over the last dim of [b, h, t, s].
  virtual LB causal_softmax(const LB& att) const { return custom_softmax(causal_mask(att)); }
  // One query position: q [b, nh, 1, d], k and v [b, nkv, s, d] -> [b, nh, 1, d].
  virtual LB attention_decode(const LB& q, const LB& k, const LB& v, float scale) const;
  // One new position straight from the projections (model.rs:207-230 at t = 1): x [b, 1, n * d]
  // becomes one row per head, rotated when a table is given (cos/sin/pos non-null), appended to
  // cache [b, n, s, d] -> [b, n, s + 1, d].
  virtual LB rope_append(const LB& cache, const LB& x, const LB* cos, const LB* sin, const LB* pos, bool interleaved) const;
  // q [b, 1, nh * d] (rotated first when a table is given), k and v [b, nkv, s, d] -> [b, 1, nh * d].
  virtual LB attention_decode_flat(const LB& q, const LB& k, const LB& v, float scale, const LB* cos, const LB* sin, const LB* pos,
                                   bool interleaved) const;

  // Caches that are written in place.  kv_cache_capacity: rows to preallocate per head for a model
  // of max_positions and this head size (0 = this device grows its caches by concatenation, as
  // model.rs:226-230 does).
  virtual size_t kv_cache_capacity(size_t max_positions, size_t head_dim) const {
    (void)max_positions;
    (void)head_dim;
    return 0;
  }
  // cache [b, n, cap, d] holds `len` rows per head; x [b, t, n * d] comes from the k or v projection
  // and is rotated at table rows pos[0] + i when a table is given.  Returns the cache with rows
  // len .. len + t - 1 written: the same storage when cap > len (in place), otherwise (cap == len,
  // the default) a new buffer [b, n, len + t, d] built with rope and cat.
  // x may be a column range of wider rows (a packed q|k|v projection): row i then starts at
  // element x_offset + i * x_row_stride of x (x_row_stride 0 = dense rows); only devices with
  // packed_projections() take that form.
  virtual LB kv_append(const LB& cache, size_t len, const LB& x, const LB* cos, const LB* sin, const LB* pos, bool interleaved, size_t x_offset = 0,
                       size_t x_row_stride = 0) const;
  // Causal attention of q [b, t, nh * d] (rotated first when a table is given) over the first s rows
  // of k and v [b, nkv, cap, d]; query i sees keys 0 .. s - t + i.  Returns [b, t, nh * d].  The
  // default composes model.rs:207-210, 231-245 and needs cap == s and, for t > 1, s == t.
  // q_offset / q_row_stride / n_heads: q as a column range of wider rows, as for kv_append
  // (n_heads = 0: taken from q's last dim).
  virtual LB attention_cached(const LB& q, const LB& k, const LB& v, size_t s, float scale, const LB* cos, const LB* sin, const LB* pos,
                              bool interleaved, size_t q_offset = 0, size_t q_row_stride = 0, size_t n_heads = 0) const;

  // x [.., k] against a matrix w [n, k] that may be stored in another dtype than x (bf16 weights under
  // f32 activations).  The default widens w with a cast in front of matmul_t (model.rs:147-158 with
  // the one dtype Device::matmul wants, ug-core/src/lib.rs:62-70).
  virtual LB linear(const LB& x, const LB& w) const;

  // Projections with their neighbours folded in.  The defaults compose matmul_t with the lazy
  // graph's own element-wise ops, exactly as model.rs:160-168, 206-208, 366-372 do.
  // packed_projections(): linear_packed gives q|k|v side by side in one buffer and kv_append /
  // attention_cached read their part of it in place.
  virtual bool packed_projections() const { return false; }
  // x [b, t, k] against up to three [n_i, k] matrices -> [b, t, n_0 + n_1 + n_2].  alpha != nullptr:
  // on rms_norm(x, *alpha, eps) instead of x (the norm in front of the projection folded in).
  virtual LB linear_packed(const LB& x, const std::vector<LB>& ws, const LB* alpha = nullptr, float eps = 0.f) const;
  // silu(x gate^T) * (x up^T), x normalised first when alpha != nullptr
  virtual LB gate_up(const LB& x, const LB& w_gate, const LB& w_up, const LB* alpha = nullptr, float eps = 0.f) const;
  // the same against one [2n, k] matrix holding the gate rows, then the up rows (several positions: one product)
  virtual LB gate_up_stacked(const LB& x, const LB& w_gate_up) const;
  // x w^T + residual
  virtual LB linear_add(const LB& x, const LB& w, const LB& residual) const;
  // Several positions with more of the layer in one schedule item (the defaults compose the ops above):
  // rms_norm(x, alpha, eps) w^T -- model.rs:65-78 in front of 206-208 --
  virtual LB linear_norm(const LB& x, const LB& alpha, float eps, const LB& w) const;
  // and the whole MLP block of model.rs:160-168 with its residual: gate_up_stacked on x (normalised first when
  // alpha != nullptr), the down projection, + residual.
  virtual LB mlp_stacked(const LB& x, const LB* alpha, float eps, const LB& w_gate_up, const LB& w_down, const LB& residual) const;

  // One decode position in one launch (devices with packed_projections()): the k and v parts of
  // the packed row qkv [b, 1, (nh + 2 nkv) d] go into row `len` of both caches (k rotated), the q
  // part attends to rows 0 .. len.  The caches are WRITTEN although they are passed as arguments:
  // they must be preallocated stores that nothing else in the same graph reads.
  virtual LB attention_step(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin,
                            const LB* pos, bool interleaved) const;

  // The same for t positions (a prompt): rows len .. len + t - 1 of both caches receive the k (rotated) and v parts
  // of the packed rows qkv [b, t, (nh + 2 nkv) d], query i attends to rows 0 .. len + i.  The default composes
  // kv_append (twice) and attention_cached; a device may fold the two appends into one launch and the three ops
  // into one schedule item.  The caches are written, as in attention_step.
  virtual LB attention_steps(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin,
                             const LB* pos, bool interleaved) const;

  // attention_steps followed by the output projection and its residual (model.rs:247 and 366-372): one schedule item on
  // devices that keep the rows between the two to themselves.  The default composes attention_steps and linear_add.
  virtual LB attention_steps_add(const LB& qkv, const LB& kcache, const LB& vcache, size_t len, size_t n_heads, float scale, const LB* cos, const LB* sin,
                                 const LB* pos, bool interleaved, const LB& w_o, const LB& residual) const;

  // Greedy step on the device (device_argmax() == true): the index of the largest value of row
  // `row` of logits [b, rows, n] is written into `token` (I32, one element, in place: the result
  // names the same storage) and recorded with the two largest values at ids[slot], vals[2 slot],
  // vals[2 slot + 1].  A decoder can then queue the next step without reading the logits back.
  virtual bool device_argmax() const { return false; }
  virtual LB argmax_into(const LB& token, const LB& logits, size_t row, const LB& ids, const LB& vals, size_t slot) const;
};

// The HIP implementation (counterpart of ug-llama/src/cuda_ops.rs).
// bf16x3: products of two or more f32 rows with a BF16 matrix split the rows into three bf16 terms and run on the
// bf16 matrix pipe (UGHIP_PRODUCT_BF16X3) instead of widening the matrix for the f32 pipe.
std::shared_ptr<Ops> hip_ops(bool bf16x3 = false);

// ug-llama/src/model.rs:10-30
struct Config {
  size_t hidden_size = 2048;
  size_t intermediate_size = 5632;
  size_t max_position_embeddings = 2048;
  size_t num_attention_heads = 32;
  size_t num_key_value_heads = 4;
  size_t num_hidden_layers = 22;
  double rms_norm_eps = 1e-5;
  bool rope_interleaved = false;
  float rope_theta = 10000.f;
  bool tie_word_embeddings = true;
  size_t vocab_size = 32000;
  size_t head_dim() const { return hidden_size / num_attention_heads; }
};

// Where the weights come from: tensors by HF name (model.rs:313-346), already f32 on the host
// (the reference always loads with `load_with_cast(.., F32, ..)`, model.rs:118,140,313).
struct WeightSource {
  virtual ~WeightSource() = default;
  virtual std::vector<float> get(const std::string& name, const std::vector<size_t>& shape) = 0;
  // The tensor as an f32 buffer on `dev`; the default uploads what get() returns.
  virtual LB load(const std::string& name, const std::vector<size_t>& shape, const ug::DevicePtr& dev);
};

// Random-init weights: N(0, std) from a counter-based generator keyed by (seed, tensor name),
// optionally rounded to bf16 (round-to-nearest-even) and widened back.
// norm_mean: the norm vectors are norm_mean + N(0, std) (checkpoints hold values near 1; BASELINE's config says N(0, 0.02), i.e. 0);
// embed_std > 0: the embedding table (and with it the tied head) is N(0, embed_std) instead of N(0, std).
std::shared_ptr<WeightSource> synthetic_weights(uint64_t seed, float std, bool round_bf16, float norm_mean = 0.f, float embed_std = 0.f);

// Weights from safetensors files, any stored dtype, delivered as f32 (model.rs:118,140,313:
// `load_with_cast(name, DType::F32, device)`); conversion happens on the device when it can.
std::shared_ptr<WeightSource> safetensors_weights(const std::vector<std::string>& paths);

// Graph builders of model.rs:32-109, usable on their own.
LB index_select(const LB& src, const LB& ids);
LB rms_norm(const LB& src, const LB& alpha, float eps);
LB repeat(const LB& lb, size_t axis, size_t n_rep);
LB softmax(const LB& src);
LB silu(const LB& src);
struct Rope {
  LB cos, sin;
  static Rope create(const Config& cfg, const ug::DevicePtr& dev);
};

// model.rs:183-198
struct Cache {
  LB prev_k, prev_v;
  // Used by the in-place mode only: rows written so far, rows allocated (0 = prev_k / prev_v have
  // exactly the rows written, the reference's representation).
  size_t len = 0, capacity = 0;
  static std::vector<Cache> create(const Config& cfg, const ug::DevicePtr& dev, size_t capacity = 0);
};

// model.rs:299-373
class Model {
 public:
  Model(const Config& cfg, bool custom_softmax, WeightSource& weights, const ug::DevicePtr& dev, std::shared_ptr<Ops> ops);
  // 0 (default): the reference's op-by-op graph.
  // 1: attention through Ops::causal_softmax (prefill) and Ops::rope_append +
  //    Ops::attention_decode_flat (one query position); caches still grow by copying.
  // 2: Ops::kv_append + Ops::attention_cached for any number of positions; with a device that
  //    preallocates (Ops::kv_cache_capacity) the caches are written in place and scores never
  //    reach memory.
  // 3: 2, and the projections through Ops::linear_packed (norm + q|k|v, norm + output head),
  //    Ops::gate_up (norm + gate, up, SwiGLU) and Ops::linear_add (o_proj / down_proj with the
  //    residual): 7 schedule items per layer and decode step on a device that fuses them.
  //    With more than one position (prefill) level 3 multiplies by q|k|v and gate|up stacked into one
  //    matrix each -- 4 products per layer instead of 7 -- and the cache appends, the attention kernel
  //    and SwiGLU read their column ranges of the wide results in place.  The stacked copies are made
  //    the first time level 3 is set on a device with packed projections and kept beside the
  //    separate matrices, which the one-position kernels stream (1.3 x the matrix bytes resident).
  void set_fused_attention(int level);
  int fused_attention() const { return fused_attention_; }
  // Keep the projection matrices and the output head in bf16 (rounded to nearest even when they
  // are not bf16 values already) and stream them in that form; activations stay f32.  The numbers
  // are those of a model whose f32 weights hold the rounded values - what a bf16 checkpoint gives
  // after load_with_cast(.., F32, ..) (model.rs:118,140,313) - because every use widens exactly:
  // inside the fused one-row projections of level 3, through a cast in front of matmul elsewhere.
  void store_matrices_bf16();
  bool bf16_matrices() const { return bf16_matrices_; }
  // Caches of the kind fwd() expects at the current fusion level.
  std::vector<Cache> new_cache() const;
  // after_layer, when given, is called with the hidden state behind every layer: a caller that realises it there
  // (schedule, compile, launch) has the device working on layer i while the graph of layer i + 1 is still being built.
  // last_position_only (fusion level 3): the head runs on the last position alone and the result is [b, 1, vocab] -- what a
  // generation loop reads of a prompt's logits; the layers and the caches are the same.
  LB fwd(const LB& tokens, const LB& pos, std::vector<Cache>& cache, const std::function<void(const LB&)>* after_layer = nullptr,
         bool last_position_only = false) const;
  const Config& config() const { return cfg_; }
  const ug::DevicePtr& device() const { return dev_; }
  const Rope& rope() const { return rope_; }
  const Ops& ops() const { return *ops_; }

 private:
  struct Layer {
    LB rms1, rms2;
    LB q_proj, k_proj, v_proj, o_proj;
    LB gate_proj, up_proj, down_proj;
    LB qkv_stacked, gate_up_stacked;  // [q; k; v] and [gate; up] by rows; invalid until level 3 asks for them
  };
  void stack_matrices();
  // residual != nullptr: the result includes the residual add; norm_first: xs still has to go
  // through the layer's RMSNorm (fusion level 3 folds both into the projections)
  LB attention(const Layer& l, const LB& xs, const LB& pos, Cache& cache, const LB* residual, bool norm_first) const;
  LB mlp(const Layer& l, const LB& xs, const LB* residual, bool norm_first) const;
  Config cfg_;
  bool custom_softmax_;
  int fused_attention_ = 0;
  ug::DevicePtr dev_;
  std::shared_ptr<Ops> ops_;
  LB embedding_, head_, ln_f_;
  bool bf16_matrices_ = false;
  Rope rope_;
  std::vector<Layer> layers_;
};

// The greedy-decode harness (the loop of ug-llama/src/main.rs:118-170): one prefill call over `prompt`, then `n_steps` greedy
// (argmax) single-token steps with the KV cache.  Returns the generated ids; timings in ms.
// Switches of the host-side loops and hooks (measurements, tests): read once per process from the environment
// (UG_LLAMA_<NAME>) and changed afterwards only through set_switch, so that the hooks running on the preparing
// thread never call getenv next to a caller that changes the environment.
enum Switch { SW_NO_FOLD_EPILOGUES, SW_NO_APPEND_PAIR, SW_VERBOSE, SW_NO_LAYER_STEPS, SW_HOST_ARGMAX, SW_NO_OVERLAP, SW_COUNT };
bool switch_on(Switch s);
bool set_switch(const std::string& name, bool on);  // false: no switch of that name ("NO_OVERLAP", "UG_LLAMA_NO_OVERLAP")

struct GenerateStats {
  double prefill_ms = 0, decode_ms = 0;
  std::vector<double> step_ms;
  std::vector<float> top1_margin;  // logit gap between the best and second-best token per step
  std::vector<float> top1_value;   // the best token's logit per step
  size_t decode_items = 0;         // schedule items (device launches) of the last single-token step
};
// forced != nullptr (n_steps ids): decode step i is fed (*forced)[i - 1] instead of the id picked at step i - 1, so that two
// devices can be compared position by position on identical inputs; the ids returned are still each step's argmax.
// Ids outside [0, vocab_size) in `prompt` or `forced` are refused (they would index the embedding table out of bounds).
std::vector<int32_t> generate_greedy(const Model& model, const std::vector<int32_t>& prompt, size_t n_steps, GenerateStats* stats,
                                     const std::vector<int32_t>* forced = nullptr);

}  // namespace ug_llama
