// Device memory, tensors and the kernel library as the native engine sees them.
//
// The engine is host code: it is compiled by the host compiler against the HIP runtime API and reaches
// the gfx950 kernels through the C entry points of libvosti_bf16.so or libvosti_f32.so, whichever the
// chosen precision names (both export the same names, so the library is picked at run time with dlopen).
// Every wrapper checks on the host that operand shapes and sizes are what the kernel's grid assumes
// before it launches: a kernel that reads out of bounds can take the GPU down.
#pragma once
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace vosti {

struct EngineError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

void hip_check(hipError_t e, const char* what);

enum class DType { BF16, F32, I32 };
inline int dtype_bytes(DType t) { return t == DType::BF16 ? 2 : 4; }
const char* dtype_name(DType t);

// Device memory that frees itself.
class DeviceBuffer {
 public:
  explicit DeviceBuffer(size_t bytes);
  ~DeviceBuffer();
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  void* data() const { return ptr_; }
  size_t bytes() const { return bytes_; }

 private:
  void* ptr_ = nullptr;
  size_t bytes_ = 0;
};

// A contiguous row-major tensor on the GPU.  `owner` keeps weights alive; activations live in the step's
// arena and have none.
struct Tensor {
  void* data = nullptr;
  DType dtype = DType::BF16;
  std::vector<int64_t> shape;
  std::shared_ptr<DeviceBuffer> owner;

  int64_t numel() const {
    int64_t n = 1;
    for (int64_t s : shape) n *= s;
    return n;
  }
  int64_t dim(int i) const { return shape.at(i < 0 ? shape.size() + i : i); }
  size_t bytes() const { return (size_t)numel() * dtype_bytes(dtype); }
  bool defined() const { return data != nullptr || numel() == 0; }
  Tensor view(std::vector<int64_t> new_shape) const;         // same elements, another shape
  Tensor rows(int64_t first, int64_t count) const;           // rows [first, first + count) of the outer axis
  std::string describe() const;
};

// Memory for one step's activations: handed out front to back, all given back at once when the step is
// over.  Blocks are only ever appended, so the same sequence of requests gets the same addresses in
// every step, which a recorded graph relies on.  Nothing is allocated while a stream is capturing.
class Arena {
 public:
  void* take(size_t bytes);
  void reset() { block_ = 0; offset_ = 0; }
  // Where the next block would be handed out.  A recorded step's results lie below the mark taken at the end
  // of its recording; after a replay the cursor goes back there, so that what is taken next (a copy of the
  // logits, say) cannot lie on top of them.
  struct Mark {
    size_t block = 0, offset = 0;
  };
  Mark mark() const { return {block_, offset_}; }
  void restore(const Mark& m) { block_ = m.block; offset_ = m.offset; }
  void forbid_growth(bool on) { frozen_ = on; }
  size_t capacity() const;

 private:
  std::vector<std::unique_ptr<DeviceBuffer>> blocks_;
  size_t block_ = 0, offset_ = 0;
  bool frozen_ = false;
};

// The kernel library of one precision.
class Kernels {
 public:
  // `lib_dir`: the folder that holds libvosti_<name>.so; name is "bf16" or "f32".
  Kernels(const std::string& lib_dir, const std::string& name);
  ~Kernels();
  Kernels(const Kernels&) = delete;

  DType dtype() const { return dtype_; }
  const std::string& name() const { return name_; }
  hipStream_t stream = nullptr;      // every launch goes here
  Arena arena;                       // where results are put

  Tensor empty(std::vector<int64_t> shape) { return empty(std::move(shape), dtype_); }
  Tensor empty(std::vector<int64_t> shape, DType t);

  Tensor embedding(const Tensor& table, const Tensor& ids);
  Tensor rmsnorm(const Tensor& x, const Tensor& w, float eps);
  Tensor add_rmsnorm(const Tensor& x, Tensor& residual, const Tensor& w, float eps);
  Tensor swiglu(const Tensor& gate_up);
  Tensor gather_rows(const Tensor& x, const Tensor& rows);
  Tensor to_f32(const Tensor& x);
  // A 32-bit tensor as elements (the tensor itself where the elements are 32-bit).
  Tensor to_elements(const Tensor& x);
  // Columns [first, first + count) of a [rows, width] tensor as a tensor of their own.
  Tensor columns(const Tensor& x, int64_t first, int64_t count);
  // dst[:, dst_first : dst_first + count] = src[:, src_first : src_first + count], rows alike.
  void copy_columns(Tensor& dst, int64_t dst_first, const Tensor& src, int64_t src_first, int64_t count);
  void rope_tables(Tensor& cos, Tensor& sin, const Tensor& inv_freq);
  // Counter-based random fill: element i is a function of (seed, i); kind 0: a sum of four 16-bit uniforms
  // scaled by p0, kind 1: p0 + u * p1.
  void fill_random(Tensor& out, uint64_t seed, int kind, float p0, float p1);
  // act @ w^T, w [out, in].  workspace: float32 scratch; with enough of it (gemm_workspace_floats) some sizes
  // take a faster route to the same bits.
  Tensor gemm(const Tensor& act, const Tensor& w, const Tensor* workspace = nullptr);
  Tensor gemm_swiglu(const Tensor& act, const Tensor& w_gate_up, const Tensor* workspace = nullptr);
  // float32 elements of workspace with which gemm / gemm_swiglu take the route through chunk sums for these
  // sizes, or 0 where that route does not exist or is the slower one.
  int64_t gemm_workspace_floats(int64_t M, int64_t rows, int64_t K, bool swiglu = false) const;
  // Head norm, rotation and cache store of [T, (nq + 2 nkv) d] rows; returns q [T, nq, d] (nq > 0).
  Tensor qkv_post(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                  const Tensor* q_w, const Tensor* k_w, float eps, const Tensor* cos, const Tensor* sin,
                  const Tensor* positions, const Tensor* slots);
  int64_t attn_scratch_floats(int items, int nq, int d, int nseg) const;
  void paged_attention(Tensor& out, const Tensor& q, const Tensor& k_cache, const Tensor& v_cache,
                       const Tensor& block_table, const Tensor& cu_q, const Tensor& k_len, const Tensor& items, int mode,
                       float scale, int window, int max_k_len, int nseg, const Tensor* scratch);
  // Token ids per row: the largest logit, or a draw at temps[r] > 0 with the uniform number unis[r].
  void sample(Tensor& out, const Tensor& logits, const Tensor* temps, const Tensor* unis, Tensor& scratch);
  int sample_scratch_words(int rows) const;
  // ---- a residual stream in 32-bit whatever the element type (stream.hip)
  // table[ids] + sinusoidal positions (entry 2i: sin(p f[i]), 2i + 1: cos(p f[i])) as floats [T, width].
  Tensor embed_sinusoid(const Tensor& table, const Tensor& ids, const Tensor& positions, const Tensor& inv_freq);
  // x (floats or elements) * rsqrt(mean(x^2) + eps) * (offset + w), as elements.
  Tensor stream_norm(const Tensor& x, const Tensor& w, float eps, float offset);
  // out = base + mult * norm(y), floats; out may be base.
  // rounded (elements of out's shape, or null): the new rows rounded to elements as well.
  void stream_norm_add(Tensor& out, const Tensor& base, const Tensor& y, const Tensor& w, float eps, float offset, float mult, Tensor* rounded = nullptr);
  // out = sum over j < n of coef[j] * states[j]; states [>= n, ...] floats.
  Tensor stream_mix(const Tensor& states, const Tensor& coef, int n);
  void softcap(Tensor& x, float cap);          // x <- cap * tanh(x / cap)
  // gemm on the columns [first, first + w.dim(1)) of act.
  Tensor gemm_columns(const Tensor& act, int64_t first, const Tensor& w);
  // qkv_post with a bias [(nq + 2 nkv) d] added to the rows first.
  Tensor qkv_post_bias(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                       const Tensor* slots, const Tensor& bias);
  // Attention with capped scores, kept first keys, a sink per head and unrounded weights (attention.hip).  block > 0
  // (without a window): positions are cut into blocks of that many, and a row sees the keys of its own block only.
  void paged_attention_capped(Tensor& out, const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, const Tensor& block_table,
                              const Tensor& cu_q, const Tensor& k_len, const Tensor& items, int mode, float scale, int window, int keep,
                              float softcap, const Tensor* sinks, int max_k_len, int nseg, const Tensor* scratch, int block = 0);
  // ---- the gated delta rule with a decay per key channel (delta.hip)
  // silu(short causal convolution) of the first taps.dim(0) columns of x, floats [T, C]; the state's tails move on.
  // first_col: where the convolution's channels start in x's rows; bias: [channels] or null.
  Tensor delta_conv(const Tensor& x, const Tensor& taps, Tensor& state, int64_t tail_offset, const Tensor& token_seq, const Tensor& cu_q,
                    const Tensor& positions, const Tensor& slots, int64_t first_col = 0, const Tensor* bias = nullptr);
  void delta_unit(Tensor& x, int64_t col0, int heads, int d, float eps, float scale);
  Tensor delta_decay(const Tensor& a, const Tensor& dt_bias, const Tensor& A_log, int H, int d);
  // Both unit norms (q at q_col times q_scale, k at k_col; G heads of d each) and the decays, in one launch; returns the decays.
  Tensor delta_prep(Tensor& x, int64_t q_col, int64_t k_col, int G, int H, int d, float unit_eps, float q_scale, const Tensor& a,
                    const Tensor& dt_bias, const Tensor& A_log);
  Tensor delta_rule(const Tensor& qkv, int q_col, int k_col, int v_col, const Tensor& decay, const Tensor& b, int64_t b_col, Tensor& state,
                    const Tensor& cu_q, const Tensor& positions, const Tensor& slots, int H, int G, int d, int dv);
  // width: the row length of the result (at least H * dv; the columns beyond are zero).
  Tensor delta_out(const Tensor& o, const Tensor& gate, const Tensor& w, int H, int dv, float eps, int64_t width);
  // ---- a stream whose embedding is scaled, sums of branches, the mean of two normed branches (stream.hip)
  Tensor embed_scaled(const Tensor& table, const Tensor& ids, float scale);
  // stream += a + b (b may be null); a and b floats or elements of the stream's shape.
  void stream_add(Tensor& stream, const Tensor& a, const Tensor* b);
  // ca * norm(a) * wa + cb * norm(b) * wb as floats; a, b elements [T, H].
  Tensor stream_pair_norm(const Tensor& a, const Tensor& wa, const Tensor& b, const Tensor& wb, float eps, float ca, float cb);
  // qkv_post whose rotation computes its angles: pair c of every q and k head turns by position * inv_freq[c] (32-bit),
  // cosine and sine times mag; no head norms.
  Tensor qkv_post_angles(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                         const Tensor& inv_freq, float mag, const Tensor& positions, const Tensor* slots);
  // The same with head norms before the rotation: q and k heads are normed over their first norm_d elements with the
  // weights q_w and k_w [norm_d] (either may be null) and eps; elements beyond norm_d (a padded head) come out zero.  The
  // rows of qkv may hold more columns than the heads' (what follows them is not read).
  Tensor qkv_post_norm_angles(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                              const Tensor* q_w, const Tensor* k_w, int norm_d, float eps, const Tensor& inv_freq, float mag, const Tensor& positions,
                              const Tensor* slots);
  // x [T, W] <- x * act(gate[:, gate_col : gate_col + W]); kind 0: the logistic function, 1: z * logistic(z).
  void gate_mul(Tensor& x, const Tensor& gate, int64_t gate_col, int kind);
  // ---- gated linear attention with a decay per key channel (delta.hip)
  // sigmoid(a + bias)^(1 / root) as floats [T, H, d]; a: elements [T, H d].
  Tensor gla_decay(const Tensor& a, const Tensor& bias, int H, int d, float root);
  // S <- diag(g) S + k v^T, o = S^T (q * q_scale) per head and token; x: element rows with q, k (H heads of d) and v (H
  // heads of dv) at the three columns.  Returns o [T, H, dv] floats; the state [slots, >= H d dv] moves on.
  Tensor gla_rule(const Tensor& x, int64_t q_col, int64_t k_col, int64_t v_col, const Tensor& decay, Tensor& state, const Tensor& cu_q,
                  const Tensor& positions, const Tensor& slots, int H, int d, int dv, float q_scale);
  // delta_out with the gate at columns [gate_col, gate_col + H dv) of a wider tensor and a choice of its activation.
  Tensor gated_head_norm(const Tensor& o, const Tensor& gate, int64_t gate_col, const Tensor& w, int H, int dv, float eps, int gate_kind, int64_t width);
  // ---- a state-space recurrence with one decay per head (ssm.hip)
  // xbc: floats [T, C] with x (H heads of P) from column 0, B (G groups of N) from b_col, C from c_col; dt: head h's step
  // size before its activation at column dt_col + h of proj (elements).  Returns y [T, H, P] floats; the state moves on.
  Tensor ssm_scan(const Tensor& xbc, int64_t b_col, int64_t c_col, const Tensor& proj, int64_t dt_col, const Tensor& dt_bias, const Tensor& A_log,
                  const Tensor& D, Tensor& state, const Tensor& cu_q, const Tensor& positions, const Tensor& slots, int H, int G, int N, int P);
  // (y * silu(z)) normed in `parts` equal parts, times w, as elements [T, width] (columns beyond y's are zero); z: the
  // columns [z_col, z_col + inner) of proj.
  Tensor ssm_gate_norm(const Tensor& y, const Tensor& proj, int64_t z_col, const Tensor& w, int parts, float eps, int64_t width);
  // ---- a mixture of experts (moe.hip)
  struct MoePlan {
    Tensor idx, wts;                            // [T, top]
    Tensor row_pair, row_token, pair_row, tile_expert;
    Tensor expert_start;                        // [experts + 1] on the GPU: every expert's first row, and the rows in use
    int top = 0, experts = 0, tile_rows = 16;   // an expert's rows are padded to whole tiles of this many
  };
  // tile_rows 16: for moe_up / moe_down; 128: for gemm_grouped, whose blocks are the plan's tiles.
  // bias: [experts], added to the logits before the choice, or null.
  MoePlan moe_route(const Tensor& h, const Tensor& router, int top, float weight_eps, int tile_rows = 16, const Tensor* bias = nullptr);
  // h W^T of every (token, choice) in the plan's rows, no activation; w [E, N, width]; result [rows, N] elements.
  Tensor moe_up_plain(const Tensor& h, const Tensor& w, const MoePlan& plan);
  // The gated activation of rows [gate: F | up: F]: min(gate, limit) * sigmoid(slope * .) * (clamp(up, +-limit) + shift), [rows, F].
  Tensor moe_glu(const Tensor& gate_up, float limit, float slope, float shift);
  // relu(h W_up^T)^2 of every (token, choice) in the plan's rows; w_up [E, ff, width]; result [rows, ff] elements.
  Tensor moe_up(const Tensor& h, const Tensor& w_up, const MoePlan& plan);
  // The chosen experts' down projections of the plan's rows, [rows, width] elements; w_down [E, width, ff].
  Tensor moe_down(const Tensor& act, const Tensor& w_down, const MoePlan& plan);
  // The weighted sum of a token's rows, floats [T, width].
  Tensor moe_sum(const Tensor& y, const MoePlan& plan, const Tensor* extra = nullptr);   // extra [T, width] elements: added last
  // act [M, K] in blocks of 128 rows, block b times the matrix block_weights[b] of w [matrices, N, K] (negative: the
  // block is skipped); [M, N] elements, the bits gemm gives for the same rows and matrix.  K in whole pairs of slabs.
  Tensor gemm_grouped(const Tensor& act, const Tensor& w, const Tensor& block_weights);
  bool gemm_grouped_takes(int64_t K) const;
  // moe_route with a choice of score: 0 as moe_route; 1: a chosen expert's weight is the logistic function of its logit.
  MoePlan moe_route_scored(const Tensor& h, const Tensor& router, int top, float weight_eps, int tile_rows, const Tensor* bias, int score_kind);
  // moe_glu for experts that read their input times the pair's weight: every row's gate and up values are multiplied by
  // its pair's weight before the clamps; moe_sum_unweighed then adds a token's rows as they are.
  Tensor moe_glu_weighed(const Tensor& gate_up, float limit, float slope, float shift, const MoePlan& plan);
  Tensor moe_sum_unweighed(const Tensor& y, const MoePlan& plan);
  // ---- attention through a latent (latent.hip)
  // norm(x[:, col : col + n]) * w as elements [T, width], the columns beyond n zero.
  Tensor norm_columns(const Tensor& x, int64_t col, int64_t n, const Tensor& w, float eps, int64_t width);
  // out[:, h * out_stride : + N] = x[:, x_col + h * x_stride : + K] W[h]^T for every head; w [H, N, K]; out [T, out_width] elements.
  void gemm_heads(Tensor& out, int64_t out_stride, const Tensor& x, int64_t x_col, int64_t x_stride, const Tensor& w);
  // The latent's norm, the rotation of the key part and of the heads' rotated query parts, and the cache store, in one
  // launch.  q_abs [T, H, D]: its columns [r, D) of every head are written.  kv_col < 0: queries only.
  void latent_post(const Tensor& proj, int64_t kv_col, const Tensor& q, int64_t q_stride, int64_t q_first, Tensor& q_abs, const Tensor* k_cache,
                   const Tensor* v_cache, int page_size, const Tensor* norm_w, float eps, const Tensor& inv_freq, bool neighbours,
                   const Tensor& positions, const Tensor* slots, int r, int dr);
  // qkv_post_norm_angles with a choice of pairs: neighbours true turns elements 2c and 2c + 1; the norms may be absent.
  Tensor qkv_post_norm_angles_paired(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                                     const Tensor* q_w, const Tensor* k_w, int norm_d, float eps, const Tensor& inv_freq, float mag, bool neighbours,
                                     const Tensor& positions, const Tensor* slots);
  // ---- linear attention with one fixed decay a head (delta.hip)
  // S <- decay[h] S + k v^T, o = S^T (q * q_scale) from the elements at the three columns of x.  decay [H] floats.  Returns o [T, H, dv] floats.
  Tensor linear_rule(const Tensor& x, int64_t q_col, int64_t k_col, int64_t v_col, const Tensor& head_decay, Tensor& state,
                     const Tensor& cu_q, const Tensor& positions, const Tensor& slots, int H, int d, int dv, float q_scale);
  // norm(o rows as a whole) * w * act(gate[:, gate_col : gate_col + n]) as elements [T, width] (zero beyond n); o: floats [T, ...] of n
  // entries a row; gate_kind 0: the logistic function, 1: z * logistic(z).
  Tensor gated_row_norm(const Tensor& o, const Tensor& gate, int64_t gate_col, const Tensor& w, float eps, int gate_kind, int64_t width);
  // x[:, first : first + count] <- silu(.) in place.
  void silu_columns(Tensor& x, int64_t first, int64_t count);
  // ---- a token's slice of a second embedding table, gated (stream.hip)
  // gelu(gate[:, 0:n]) * table[ids, first : first + n] as elements [T, gate.dim(1)], zero beyond n.
  Tensor side_gate(const Tensor& gate, const Tensor& table, const Tensor& ids, int64_t first, int64_t n);
  void relu_square(Tensor& x);                 // x <- max(x, 0)^2
  int segment_keys() const { return segment_keys_; }
  int item_rows() const { return item_rows_; }

 private:
  void call(int rc) const;
  void expect(const Tensor& t, const char* what, DType dtype, std::vector<int64_t> shape = {}) const;
  int norm_weight(const Tensor& w, const char* what, int64_t n) const;   // 1 if the weight is float32
  bool split(Tensor& out, const Tensor& act, const Tensor& w, bool swiglu, const Tensor* workspace);

  std::string name_;
  DType dtype_;
  void* handle_ = nullptr;
  int segment_keys_ = 0, item_rows_ = 0;
  struct Fn;
  std::unique_ptr<Fn> fn_;
};

}  // namespace vosti
