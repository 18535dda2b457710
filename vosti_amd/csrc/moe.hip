// A mixture of small feed-forward experts, each token through its `top` best of E: the router, the plan that sorts
// (token, choice) pairs by expert into tiles of rows, the two projections as grouped products on the matrix unit,
// and the weighted sum of a token's experts.
//
//   z = W_router h (32-bit sums of the elements' exact products);  s = softmax(z) over all experts;  the `top` largest
//   s (the lower index wins a tie);  weight_k = s_k / (sum of the chosen s + weight_eps);
//   out = sum over the chosen k, in the order they were chosen, of weight_k * W_down[e_k] act(W_up[e_k] h),
//   act(u) = max(u, 0)^2.
//
// A row of a grouped product depends on its own inputs only, and its sums have the order of this library's other
// matrix products, so a token's result does not depend on which other tokens share its tile or where the plan put it,
// and a caller may run an expert's rows through those products instead (many rows an expert) to the same bits.
#include <algorithm>

#include "common.h"
#include "mma.h"
#include "vec.h"

#define MOE_TILE 16          // rows of a tile: pairs of one expert
#define MOE_ROUTE_TOKENS 8   // tokens a router workgroup shares an expert's weights among

// Router logits z [T, E] floats.  A workgroup of four waves takes MOE_ROUTE_TOKENS tokens and one expert; the waves
// split the row's 16-byte vectors (vector v goes to wave (v / 64) % 4, lane v % 64), a lane adds its products in ascending
// order (fused multiply-adds), a butterfly follows over the lanes and the four waves' sums are added in wave order: the
// order depends on the width alone.
// bias: one number an expert that is added to its logit (elements or floats), or null.
__global__ __launch_bounds__(256) void moe_logits_kernel(float* __restrict__ z, const elem_t* __restrict__ h, const elem_t* __restrict__ router,
                                                         int T, int W, int E, const void* __restrict__ bias, int bias_is_f32) {
  __shared__ float part[4][MOE_ROUTE_TOKENS];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t0 = blockIdx.x * MOE_ROUTE_TOKENS, e = blockIdx.y;
  float acc[MOE_ROUTE_TOKENS];
#pragma unroll
  for (int i = 0; i < MOE_ROUTE_TOKENS; ++i) acc[i] = 0.f;
  const elem_t* wr = router + (int64_t)e * W;
#pragma unroll 2
  for (int c = threadIdx.x * VK_VEC; c < W; c += 256 * VK_VEC) {
    float wv[VK_VEC];
    load_elems(wr + c, wv);
#pragma unroll
    for (int i = 0; i < MOE_ROUTE_TOKENS; ++i) {
      float hv[VK_VEC];
      load_elems(h + (int64_t)min(t0 + i, T - 1) * W + c, hv);
#pragma unroll
      for (int j = 0; j < VK_VEC; ++j) acc[i] = __builtin_fmaf(hv[j], wv[j], acc[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < MOE_ROUTE_TOKENS; ++i) {
    const float v = wave_sum_xor(acc[i]);
    if (lane == 0) part[wave][i] = v;
  }
  __syncthreads();
  if (threadIdx.x < MOE_ROUTE_TOKENS && t0 + (int)threadIdx.x < T) {
    float v = part[0][threadIdx.x];
    v = v + part[1][threadIdx.x];
    v = v + part[2][threadIdx.x];
    v = v + part[3][threadIdx.x];
    if (bias != nullptr) v = v + load_weight(bias, bias_is_f32, e);
    z[(int64_t)(t0 + threadIdx.x) * E + e] = v;
  }
}

// The choice: idx [T, top] int32, wts [T, top] floats from the logits.  One wave per token, four tokens a workgroup.
// score 0: the softmax over all experts, the chosen scores divided by their sum plus weight_eps; score 1: the logistic
// function of every logit, the chosen scores as they are (the order of the scores is the order of the logits either way).
__global__ __launch_bounds__(256) void moe_choose_kernel(int32_t* __restrict__ idx, float* __restrict__ wts, const float* __restrict__ logits,
                                                         int T, int E, int top, float weight_eps, int score_kind) {
  extern __shared__ float scores[];      // [4][E]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  float* z = scores + wave * E;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) {
    z[e] = logits[(int64_t)t * E + e];
    mx = fmaxf(mx, z[e]);
  }
  mx = wave_max_xor(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) {
    const float p = score_kind == 1 ? 1.f / (1.f + expf(-z[e])) : expf(z[e] - mx);
    z[e] = p;
    sum = sum + p;
  }
  sum = score_kind == 1 ? 1.f : wave_sum_xor(sum);
  // The largest score `top` times; a chosen one is marked with -1 (scores are positive or zero).
  float chosen_sum = 0.f;
  float my_w = 0.f;
  int my_e = 0;
  for (int k = 0; k < top; ++k) {
    float best = -2.f;
    int best_e = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = z[e];
      if (v > best) { best = v; best_e = e; }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const float ov = __shfl_xor(best, off, VK_WAVE);
      const int oe = __shfl_xor(best_e, off, VK_WAVE);
      if (ov > best || (ov == best && oe < best_e)) { best = ov; best_e = oe; }
    }
    const float score = best / sum;
    chosen_sum = chosen_sum + score;
    if (lane == k % 64 && k < 64) { my_w = score; my_e = best_e; }
    if (k >= 64 && lane == 0) { idx[(int64_t)t * top + k] = best_e; wts[(int64_t)t * top + k] = score; }
    if (lane == 0) z[best_e] = -1.f;
    __builtin_amdgcn_wave_barrier();
  }
  const float denom = score_kind == 1 ? 1.f : chosen_sum + weight_eps;
  if (lane < top) {
    idx[(int64_t)t * top + lane] = my_e;
    wts[(int64_t)t * top + lane] = my_w / denom;
  }
  for (int k = 64 + lane; k < top; k += 64) wts[(int64_t)t * top + k] = wts[(int64_t)t * top + k] / denom;
}

// The plan, by one workgroup.  counts the pairs of every expert, gives expert e the rows [start_e, start_e + tile_rows *
// ceil(count_e / tile_rows)) and every pair a row among its expert's (in no fixed order: a row's result does not depend on
// its place).  row_pair [max_rows]: the pair (token * top + choice) of a row, or -1; row_token [max_rows]: the row's
// token (0 for a row without a pair); pair_row [pairs]; tile_expert [max_tiles]: the expert of a tile, or -1 beyond the
// last; expert_start [E + 1]: the first row of every expert, and the rows in use.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ idx, int32_t* __restrict__ row_pair,
                                                        int32_t* __restrict__ row_token, int32_t* __restrict__ pair_row,
                                                        int32_t* __restrict__ tile_expert, int32_t* __restrict__ expert_start, int pairs, int top,
                                                        int E, int max_tiles, int tile_rows) {
  extern __shared__ int32_t plan[];      // [E] counts, then [E] cursors
  int32_t* count = plan;
  int32_t* cursor = plan + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  for (int r = threadIdx.x; r < max_tiles * tile_rows; r += blockDim.x) {
    row_pair[r] = -1;
    row_token[r] = 0;
  }
  for (int i = threadIdx.x; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) atomicAdd(&count[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int tile = 0;
    for (int e = 0; e < E; ++e) {
      const int n = (count[e] + tile_rows - 1) / tile_rows;
      cursor[e] = tile * tile_rows;
      expert_start[e] = tile * tile_rows;
      for (int j = 0; j < n; ++j) tile_expert[tile + j] = e;
      tile += n;
    }
    expert_start[E] = tile * tile_rows;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int row = atomicAdd(&cursor[idx[i]], 1);
    row_pair[row] = i;
    row_token[row] = i / top;
    pair_row[i] = row;
  }
}

// One tile of 16 rows and 16 output features a workgroup: out[row, f] = sum over k of x[row, k] * w[expert][f, k], in
// the order of this library's other products: the reduction axis in chunks of MOE_KC elements, a chunk's products added
// from zero over ascending slabs of 64 bytes with the weights as first operand, the chunk sums added to a zero total in
// chunk order.  The workgroup's eight waves take chunks wave, wave + 8, ... with MOE_W slabs in flight each, and the
// chunk sums meet in LDS.  UP: the rows' inputs are the tokens' (row_token) and the output is the square of max(., 0) of
// the sum rounded to the element type, as elements; else the inputs are the rows themselves and the output the sum, as
// elements.
#define MOE_KC 512
#define MOE_KC_SLABS (MOE_KC / VK_SLAB)
#define MOE_WAVES 8
#define MOE_W 4
// MODE 0: the rows themselves are the inputs (down); 1: the rows' tokens, with the squared-relu activation; 2: the rows'
// tokens, the sum as it is (an activation of two products' outputs follows in a launch of its own).
template <int MODE>
__global__ __launch_bounds__(64 * MOE_WAVES) void moe_gemm_kernel(elem_t* __restrict__ out, int64_t ldo, const elem_t* __restrict__ x, int64_t ldx,
                                                                  const elem_t* __restrict__ w, int64_t expert_stride,
                                                                  const int32_t* __restrict__ row_pair, const int32_t* __restrict__ row_token,
                                                                  const int32_t* __restrict__ tile_expert, int N, int K) {
  __shared__ f32x4 part[MOE_WAVES][64];
  const int tile = blockIdx.y;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kq = lane >> 4;
  const int f0 = blockIdx.x * 16;
  const int row = tile * MOE_TILE + r16;
  const bool x_ok = row_pair[row] >= 0;
  constexpr bool UP = MODE != 0;
  const elem_t* xr = x + (int64_t)(UP ? row_token[row] : row) * ldx + kq * VK_VEC;
  const bool w_ok = f0 + r16 < N;
  const elem_t* wr = w + (int64_t)e * expert_stride + (int64_t)(w_ok ? f0 + r16 : 0) * K + kq * VK_VEC;
  const int nchunks = (K + MOE_KC - 1) / MOE_KC;
  const int rounds = (nchunks + MOE_WAVES - 1) / MOE_WAVES;

  frag_t wbuf[MOE_W], xbuf[MOE_W];
  auto issue = [&](int c, int s, int slot) {
    const int k = c * MOE_KC + s * VK_SLAB;
    const bool k_ok = k + kq * VK_VEC < K;
    wbuf[slot] = load_frag(wr + k, w_ok && k_ok);
    xbuf[slot] = load_frag(xr + k, x_ok && k_ok);
  };
  int c = wave;
  if (c < nchunks) {
#pragma unroll
    for (int i = 0; i < MOE_W; ++i) issue(c, i, i);
  }
  f32x4 total = {0.f, 0.f, 0.f, 0.f};
  for (int round = 0; round < rounds; ++round, c += MOE_WAVES) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (c < nchunks) {
      const int cn = c + MOE_WAVES;
      const bool has_next = cn < nchunks;
#pragma unroll
      for (int i = 0; i < MOE_KC_SLABS; ++i) {
        const int slot = i % MOE_W;
        const frag_t fw = wbuf[slot], fx = xbuf[slot];
        if (i + MOE_W < MOE_KC_SLABS) issue(c, i + MOE_W, slot);
        else if (has_next) issue(cn, i + MOE_W - MOE_KC_SLABS, slot);
        acc = mma_slab(fw, fx, acc);
      }
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0) {
      for (int w2 = 0; w2 < MOE_WAVES; ++w2) {
        if (round * MOE_WAVES + w2 < nchunks) {
          const f32x4 p = part[w2][lane];
          total.x = total.x + p.x; total.y = total.y + p.y; total.z = total.z + p.z; total.w = total.w + p.w;
        }
      }
    }
    __syncthreads();
  }
  // Lane l holds features f0 + 4 * (l / 16) + i for row l % 16.
  if (wave != 0 || !x_ok) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int f = f0 + kq * 4 + i;
    if (f >= N) continue;
    float v = total[i];
    if (MODE == 1) {
      const float rl = fmaxf(round_to_elem(v), 0.f);
      v = rl * rl;
    }
    out[(int64_t)row * ldo + f] = from_f32<elem_t>(v);
  }
}

// x <- max(x, 0)^2, element by element: the experts' activation on a product that was left as elements.  A thread
// takes a 16-byte vector (n in whole vectors).
__global__ __launch_bounds__(256) void moe_relu_square_kernel(elem_t* x, int64_t nvec) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nvec) return;
  float v[VK_VEC];
  load_elems(x + i * VK_VEC, v);
#pragma unroll
  for (int j = 0; j < VK_VEC; ++j) {
    const float rl = fmaxf(v[j], 0.f);
    v[j] = rl * rl;
  }
  store_elems(x + i * VK_VEC, v);
}

// A gated expert's activation between its two products: row r of `in` holds the gate's F outputs and, from column F on,
// the up projection's; y = g * sigmoid(slope * g) * (u + shift) with g = min(gate, limit) and u = clamp(up, -limit, limit),
// in 32-bit, as elements [rows, F].  A thread takes a 16-byte vector (F in whole vectors).
// row_pair / wts (both or neither): row r's gate and up values are multiplied by the weight of the row's (token, choice) pair
// before they are clamped, which is what an expert computes that reads its input times that weight; a row without a pair
// gives zeros.
__global__ __launch_bounds__(256) void moe_glu_kernel(elem_t* __restrict__ out, const elem_t* __restrict__ in, int64_t rows, int F, float limit,
                                                      float slope, float shift, const int32_t* __restrict__ row_pair, const float* __restrict__ wts) {
  const int per = F / VK_VEC;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * per) return;
  const int64_t r = i / per;
  const int c = (int)(i - r * per) * VK_VEC;
  float g[VK_VEC], u[VK_VEC];
  float rw = 1.f;
  if (row_pair != nullptr) {
    const int pair = row_pair[r];
    if (pair < 0) {
#pragma unroll
      for (int j = 0; j < VK_VEC; ++j) g[j] = 0.f;
      store_elems(out + r * F + c, g);
      return;
    }
    rw = wts[pair];
  }
  load_elems(in + r * 2 * F + c, g);
  load_elems(in + r * 2 * F + F + c, u);
#pragma unroll
  for (int j = 0; j < VK_VEC; ++j) {
    const float gc = fminf(g[j] * rw, limit), uc = fminf(fmaxf(u[j] * rw, -limit), limit);
    g[j] = (gc / (1.f + expf(-slope * gc))) * (uc + shift);
  }
  store_elems(out + r * F + c, g);
}

// out[t, c] = sum over k < top, ascending, of wts[t, k] * y[pair_row[t * top + k], c] (wts null: every weight 1), from zero; then + extra[t, c]
// (elements, the output of an expert that every token uses) where there is one.
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ out, const elem_t* __restrict__ y, const float* __restrict__ wts,
                                                          const int32_t* __restrict__ pair_row, int W, int top, const elem_t* __restrict__ extra) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += gridDim.y * 256) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc = acc + (wts != nullptr ? wts[(int64_t)t * top + k] : 1.f) * to_f32(y[(int64_t)pair_row[(int64_t)t * top + k] * W + c]);
    if (extra != nullptr) acc = acc + to_f32(extra[(int64_t)t * W + c]);
    out[(int64_t)t * W + c] = acc;
  }
}

extern "C" {

// Tiles that the plan may need for T tokens: every pair, and up to tile_rows - 1 rows of padding an expert that got any.
int vk_moe_max_tiles(int T, int top, int E, int tile_rows) {
  const int64_t pairs = (int64_t)T * top;
  const int64_t busy = std::min<int64_t>(E, pairs);
  return (int)((pairs + busy * (tile_rows - 1)) / tile_rows);
}

// logits: scratch [T, E] floats.  bias [E] (elements, or floats with bias_is_f32) or null.
static int route_launch(int32_t* idx, float* wts, float* logits, const elem_t* h, const elem_t* router, const void* bias, int bias_is_f32, int T, int W,
                        int E, int top, float weight_eps, hipStream_t st, int score_kind = 0) {
  VK_REQUIRE(T >= 0 && W > 0 && W % VK_VEC == 0 && E > 0 && top > 0 && top <= E && E <= 4096,
             "router: bad sizes T=%d W=%d E=%d top=%d (the width in whole 16-byte vectors, at most 4096 experts)", T, W, E, top);
  VK_REQUIRE(((uintptr_t)h % 16) == 0 && ((uintptr_t)router % 16) == 0, "router: operands must be 16-byte aligned");
  if (T == 0) return 0;
  moe_logits_kernel<<<dim3((T + MOE_ROUTE_TOKENS - 1) / MOE_ROUTE_TOKENS, E), 256, 0, st>>>(logits, h, router, T, W, E, bias, bias_is_f32);
  if (vk_check_launch("router (logits)")) return 1;
  moe_choose_kernel<<<(T + 3) / 4, 256, (size_t)4 * E * sizeof(float), st>>>(idx, wts, logits, T, E, top, weight_eps, score_kind);
  return vk_check_launch("router (choice)");
}

int vk_moe_route(int32_t* idx, float* wts, float* logits, const elem_t* h, const elem_t* router, int T, int W, int E, int top, float weight_eps,
                 hipStream_t st) {
  return route_launch(idx, wts, logits, h, router, nullptr, 0, T, W, E, top, weight_eps, st);
}

// The same with a bias an expert on the logits, which both the choice and the weights see.  With weight_eps 0 the weights
// are the softmax over the chosen logits alone: exp(z_k) / sum over the chosen exp(z_j), whatever the others are.
int vk_moe_route_bias(int32_t* idx, float* wts, float* logits, const elem_t* h, const elem_t* router, const void* bias, int bias_is_f32, int T, int W,
                      int E, int top, float weight_eps, hipStream_t st) {
  VK_REQUIRE(bias != nullptr, "router: the bias is missing");
  return route_launch(idx, wts, logits, h, router, bias, bias_is_f32, T, W, E, top, weight_eps, st);
}

// The same with a choice of score: 0 is vk_moe_route (vk_moe_route_bias with a bias), 1 gives every chosen expert the
// logistic function of its logit as its weight, not divided by anything.  bias may be null.
int vk_moe_route_scored(int32_t* idx, float* wts, float* logits, const elem_t* h, const elem_t* router, const void* bias, int bias_is_f32, int T, int W,
                        int E, int top, float weight_eps, int score_kind, hipStream_t st) {
  VK_REQUIRE(score_kind == 0 || score_kind == 1, "router: score kind %d", score_kind);
  return route_launch(idx, wts, logits, h, router, bias, bias_is_f32, T, W, E, top, weight_eps, st, score_kind);
}

int vk_moe_plan(const int32_t* idx, int32_t* row_pair, int32_t* row_token, int32_t* pair_row, int32_t* tile_expert, int32_t* expert_start, int T,
                int top, int E, int tile_rows, hipStream_t st) {
  VK_REQUIRE(T >= 0 && top > 0 && E > 0 && E <= 4096 && tile_rows > 0, "expert plan: bad sizes T=%d top=%d E=%d", T, top, E);
  if (T == 0) return 0;
  moe_plan_kernel<<<1, 1024, (size_t)2 * E * sizeof(int32_t), st>>>(idx, row_pair, row_token, pair_row, tile_expert, expert_start, T * top, top, E,
                                                                    vk_moe_max_tiles(T, top, E, tile_rows), tile_rows);
  return vk_check_launch("expert plan");
}

// act [max_rows, ldo] elements = relu(x[token of row] . w_up[expert of row])^2; w_up [E, N, K].
int vk_moe_up(elem_t* act, int64_t ldo, const elem_t* x, int64_t ldx, const elem_t* w_up, const int32_t* row_pair, const int32_t* row_token,
              const int32_t* tile_expert, int T, int top, int E, int N, int K, hipStream_t st) {
  VK_REQUIRE(T >= 0 && top > 0 && E > 0 && N > 0 && K > 0 && K % VK_VEC == 0 && ldx % VK_VEC == 0 && ldx >= K && ldo >= N,
             "experts (up): bad sizes N=%d K=%d (K in whole 16-byte vectors)", N, K);
  VK_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w_up % 16) == 0, "experts (up): operands must be 16-byte aligned");
  if (T == 0) return 0;
  const int tiles = vk_moe_max_tiles(T, top, E, MOE_TILE);
  VK_REQUIRE(tiles <= 65535, "experts (up): too many tiles for one launch");
  moe_gemm_kernel<1><<<dim3((N + 15) / 16, tiles), 64 * MOE_WAVES, 0, st>>>(act, ldo, x, ldx, w_up, (int64_t)N * K, row_pair, row_token, tile_expert,
                                                                               N, K);
  return vk_check_launch("experts (up)");
}

// act [max_rows, ldo] elements = x[token of row] . w[expert of row], no activation; w [E, N, K].
int vk_moe_up_plain(elem_t* act, int64_t ldo, const elem_t* x, int64_t ldx, const elem_t* w, const int32_t* row_pair, const int32_t* row_token,
                    const int32_t* tile_expert, int T, int top, int E, int N, int K, hipStream_t st) {
  VK_REQUIRE(T >= 0 && top > 0 && E > 0 && N > 0 && K > 0 && K % VK_VEC == 0 && ldx % VK_VEC == 0 && ldx >= K && ldo >= N,
             "experts (up): bad sizes N=%d K=%d (K in whole 16-byte vectors)", N, K);
  VK_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "experts (up): operands must be 16-byte aligned");
  if (T == 0) return 0;
  const int tiles = vk_moe_max_tiles(T, top, E, MOE_TILE);
  VK_REQUIRE(tiles <= 65535, "experts (up): too many tiles for one launch");
  moe_gemm_kernel<2><<<dim3((N + 15) / 16, tiles), 64 * MOE_WAVES, 0, st>>>(act, ldo, x, ldx, w, (int64_t)N * K, row_pair, row_token, tile_expert, N, K);
  return vk_check_launch("experts (up)");
}

// out [rows, F] elements from in [rows, 2 F]: the gated activation with clamped inputs (moe_glu_kernel).
int vk_moe_glu(elem_t* out, const elem_t* in, int64_t rows, int F, float limit, float slope, float shift, hipStream_t st) {
  VK_REQUIRE(rows >= 0 && F > 0 && F % VK_VEC == 0 && limit > 0.f && ((uintptr_t)out % 16) == 0 && ((uintptr_t)in % 16) == 0,
             "experts (gated activation): bad sizes rows=%lld F=%d (whole 16-byte vectors)", (long long)rows, F);
  if (rows == 0) return 0;
  const int64_t n = rows * (F / VK_VEC);
  moe_glu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(out, in, rows, F, limit, slope, shift, nullptr, nullptr);
  return vk_check_launch("experts (gated activation)");
}

// The same for experts that read their input times the pair's weight: row r's gate and up values are multiplied by
// wts[row_pair[r]] before the clamps (W (w h) = w (W h)); rows without a pair come out zero.
int vk_moe_glu_weighed(elem_t* out, const elem_t* in, int64_t rows, int F, float limit, float slope, float shift, const int32_t* row_pair,
                       const float* wts, hipStream_t st) {
  VK_REQUIRE(rows >= 0 && F > 0 && F % VK_VEC == 0 && limit > 0.f && ((uintptr_t)out % 16) == 0 && ((uintptr_t)in % 16) == 0,
             "experts (gated activation): bad sizes rows=%lld F=%d (whole 16-byte vectors)", (long long)rows, F);
  VK_REQUIRE(row_pair != nullptr && wts != nullptr, "experts (gated activation): the rows' pairs and weights are missing");
  if (rows == 0) return 0;
  const int64_t n = rows * (F / VK_VEC);
  moe_glu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(out, in, rows, F, limit, slope, shift, row_pair, wts);
  return vk_check_launch("experts (gated activation)");
}

// y [max_rows, N] elements = act[row] . w_down[expert of row]; w_down [E, N, K]; act rows of length lda >= K.
int vk_moe_down(elem_t* y, const elem_t* act, int64_t lda, const elem_t* w_down, const int32_t* row_pair, const int32_t* tile_expert, int T,
                int top, int E, int N, int K, hipStream_t st) {
  VK_REQUIRE(T >= 0 && top > 0 && E > 0 && N > 0 && K > 0 && K % VK_VEC == 0 && lda % VK_VEC == 0 && lda >= K,
             "experts (down): bad sizes N=%d K=%d (K in whole 16-byte vectors)", N, K);
  VK_REQUIRE(((uintptr_t)act % 16) == 0 && ((uintptr_t)w_down % 16) == 0, "experts (down): operands must be 16-byte aligned");
  if (T == 0) return 0;
  const int tiles = vk_moe_max_tiles(T, top, E, MOE_TILE);
  VK_REQUIRE(tiles <= 65535, "experts (down): too many tiles for one launch");
  moe_gemm_kernel<0><<<dim3((N + 15) / 16, tiles), 64 * MOE_WAVES, 0, st>>>(y, N, act, lda, w_down, (int64_t)N * K, row_pair, nullptr, tile_expert,
                                                                                N, K);
  return vk_check_launch("experts (down)");
}

int vk_moe_relu_square(elem_t* x, int64_t n, hipStream_t st) {
  VK_REQUIRE(n >= 0 && n % VK_VEC == 0 && ((uintptr_t)x % 16) == 0, "experts (activation): whole 16-byte vectors are needed");
  if (n == 0) return 0;
  const int64_t nvec = n / VK_VEC;
  moe_relu_square_kernel<<<(unsigned)((nvec + 255) / 256), 256, 0, st>>>(x, nvec);
  return vk_check_launch("experts (activation)");
}

static int combine_launch(float* out, const elem_t* y, const float* wts, const int32_t* pair_row, const elem_t* extra, int T, int W, int top,
                          hipStream_t st) {
  VK_REQUIRE(T >= 0 && W > 0 && top > 0, "experts (sum): bad sizes T=%d W=%d top=%d", T, W, top);
  if (T == 0) return 0;
  const int by = std::min((W + 255) / 256, 64);
  moe_combine_kernel<<<dim3(T, by), 256, 0, st>>>(out, y, wts, pair_row, W, top, extra);
  return vk_check_launch("experts (sum)");
}

int vk_moe_combine(float* out, const elem_t* y, const float* wts, const int32_t* pair_row, int T, int W, int top, hipStream_t st) {
  return combine_launch(out, y, wts, pair_row, nullptr, T, W, top, st);
}

// The same, and extra [T, W] (elements) is added to every token's sum last.
int vk_moe_combine_add(float* out, const elem_t* y, const float* wts, const int32_t* pair_row, const elem_t* extra, int T, int W, int top,
                       hipStream_t st) {
  VK_REQUIRE(extra != nullptr, "experts (sum): the output to add is missing");
  return combine_launch(out, y, wts, pair_row, extra, T, W, top, st);
}

}  // extern "C"
