// The gated delta rule with one decay per head and key channel, and what stands around it: the short causal
// convolution with its carried inputs, the unit norms, the decays, the recurrence over a state that is carried from
// step to step in 32-bit, and the gated norm of its read-out.
//
// Per head, with the state S [dim, vdim] (rows are key channels), for every token in order:
//   S <- diag(g) S;  u = beta * (v - S^T k);  S <- S + k u^T;  o = S^T q
// so that the read-out sees the token's own write.  g = exp(-exp(A_log) * softplus(a + dt_bias)), beta = sigmoid(b).
// Everything here is 32-bit; the projections that feed it (a, b, the convolutions' inputs) arrive as elements.
//
// A sequence's tokens are walked in order by one workgroup per (sequence, head, block of value columns), so the sums
// of a token do not depend on how the sequence was cut into steps or on what else is in the batch: the state that a
// step leaves in memory is the state the next step starts from, bit for bit.
#include "common.h"
#include "vec.h"

#define DELTA_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

// y[t, c] = silu(sum over j of taps[c, j] * x[t - (K - 1) + j, c]): inputs before the step's first token come from the
// sequence's carried tail (its last K - 1 inputs, oldest first), or are zero when the sequence starts here.
__global__ __launch_bounds__(256) void delta_conv_kernel(float* __restrict__ y, const elem_t* __restrict__ x, int64_t ldx,
                                                         const elem_t* __restrict__ taps, const float* __restrict__ state,
                                                         int64_t state_stride, int64_t tail_offset, const int32_t* __restrict__ token_seq,
                                                         const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                                         const int32_t* __restrict__ slots, int C, int K,
                                                         const elem_t* __restrict__ bias) {
  const int t = blockIdx.x;
  const int s = token_seq[t];
  const int first = cu_q[s], i = t - first;
  const bool fresh = positions[first] == 0;
  const float* tail = state + (int64_t)slots[s] * state_stride + tail_offset;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float acc = bias != nullptr ? to_f32(bias[c]) : 0.f;
    for (int j = 0; j < K; ++j) {
      const int li = i - (K - 1) + j;
      float v;
      if (li >= 0) v = to_f32(x[(int64_t)(first + li) * ldx + c]);
      else v = fresh ? 0.f : tail[(int64_t)(K - 1 + li) * C + c];
      acc = acc + to_f32(taps[(int64_t)c * K + j]) * v;
    }
    y[(int64_t)t * C + c] = silu_f(acc);
  }
}

// The tail after the step: the last K - 1 inputs of the sequence, oldest first.
__global__ __launch_bounds__(256) void delta_conv_tail_kernel(const elem_t* __restrict__ x, int64_t ldx, float* state,
                                                              int64_t state_stride, int64_t tail_offset,
                                                              const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                                              const int32_t* __restrict__ slots, int C, int K) {
  const int s = blockIdx.x;
  const int first = cu_q[s], n = cu_q[s + 1] - first;
  const bool fresh = positions[first] == 0;
  float* tail = state + (int64_t)slots[s] * state_stride + tail_offset;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    float keep[DELTA_MAX_TAPS];
#pragma unroll
    for (int r = 0; r < DELTA_MAX_TAPS; ++r) {
      if (r < K - 1) {
        const int li = n - (K - 1) + r;
        keep[r] = li >= 0 ? to_f32(x[(int64_t)(first + li) * ldx + c]) : (fresh ? 0.f : tail[(int64_t)(K - 1 + li) * C + c]);
      }
    }
#pragma unroll
    for (int r = 0; r < DELTA_MAX_TAPS; ++r)
      if (r < K - 1) tail[(int64_t)r * C + c] = keep[r];
  }
}

// x[t, head, :] <- x / sqrt(sum(x^2) + eps) * scale for `heads` heads of d channels that start at column col0 of rows
// of length ld.  One wave per (token, head); lane l owns channels l, l + 64, ...
__global__ __launch_bounds__(64) void delta_unit_kernel(float* x, int64_t ld, int col0, int heads, int d, float eps, float scale) {
  const int t = blockIdx.x / heads, h = blockIdx.x - t * heads;
  float* row = x + (int64_t)t * ld + col0 + (int64_t)h * d;
  float part = 0.f;
  for (int c = threadIdx.x; c < d; c += 64) part = part + row[c] * row[c];
  const float r = scale / sqrtf(wave_sum_xor(part) + eps);
  for (int c = threadIdx.x; c < d; c += 64) row[c] = row[c] * r;
}

// g[t, h, c] = exp(-exp(A_log[h]) * softplus(a[t, h * d + c] + dt_bias[h * d + c])).
__global__ __launch_bounds__(256) void delta_decay_kernel(float* __restrict__ g, const elem_t* __restrict__ a, const void* __restrict__ dt_bias,
                                                          const void* __restrict__ A_log, int w_is_f32, int d, int HD, int64_t numel) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= numel) return;
  const int col = (int)(e % HD);
  const float z = to_f32(a[e]) + load_weight(dt_bias, w_is_f32, col);
  const float sp = z > 20.f ? z : log1pf(expf(z));
  g[e] = expf(-expf(load_weight(A_log, w_is_f32, col / d)) * sp);
}

// g[t, c] = sigmoid(a[t, c] + bias[c])^inv_root, as exp(-softplus(-z) * inv_root): the logarithm of the logistic function
// is -softplus(-z), so the power needs no logarithm of a number near 1.
__global__ __launch_bounds__(256) void gla_decay_kernel(float* __restrict__ g, const elem_t* __restrict__ a, int64_t lda, const void* __restrict__ bias,
                                                        int w_is_f32, int HD, float inv_root, int64_t numel) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= numel) return;
  const int64_t t = e / HD;
  const int col = (int)(e - t * HD);
  const float z = -(to_f32(a[t * lda + col]) + load_weight(bias, w_is_f32, col));
  const float sp = z > 20.f ? z : log1pf(expf(z));
  g[e] = expf(-sp * inv_root);
}

// The two unit norms and the decays of a token in one launch: workgroup (token, j) is q's head j, k's head j - G, or
// the decays of head j - 2 G; the arithmetic is delta_unit_kernel's and delta_decay_kernel's.
__global__ __launch_bounds__(64) void delta_prep_kernel(float* x, int64_t ld, int q_col, int k_col, int G, int H, int d, float unit_eps,
                                                        float q_scale, float* __restrict__ g, const elem_t* __restrict__ a,
                                                        const void* __restrict__ dt_bias, const void* __restrict__ A_log, int w_is_f32) {
  const int per = 2 * G + H;
  const int t = blockIdx.x / per, j = blockIdx.x - t * per;
  if (j < 2 * G) {
    const bool is_q = j < G;
    float* row = x + (int64_t)t * ld + (is_q ? q_col + (int64_t)j * d : k_col + (int64_t)(j - G) * d);
    float part = 0.f;
    for (int c = threadIdx.x; c < d; c += 64) part = part + row[c] * row[c];
    const float r = (is_q ? q_scale : 1.f) / sqrtf(wave_sum_xor(part) + unit_eps);
    for (int c = threadIdx.x; c < d; c += 64) row[c] = row[c] * r;
  } else {
    const int h = j - 2 * G;
    const float rate = expf(load_weight(A_log, w_is_f32, h));
    for (int c = threadIdx.x; c < d; c += 64) {
      const int64_t e = ((int64_t)t * H + h) * d + c;
      const float z = to_f32(a[e]) + load_weight(dt_bias, w_is_f32, h * d + c);
      const float sp = z > 20.f ? z : log1pf(expf(z));
      g[e] = expf(-rate * sp);
    }
  }
}

// The recurrence.  A workgroup of four waves takes 4 * 64 / R value columns of one (sequence, head); a column's state
// is spread over R neighbouring lanes, lane r of them holding DR consecutive key channels in registers (4 for key sizes up to 256: more lanes
// a column mean more waves and shorter sums a token).  The
// inputs of a chunk of tokens (q, k and the decays of the head, the columns' v, beta) are brought into LDS by the whole
// workgroup, the next chunk's while this one is computed (global memory -> registers before the chunk's work, registers
// -> the other LDS buffer after it, one barrier a chunk), so that the walk over the tokens waits for LDS only.  The two
// sums of a token run over a lane's channels in ascending order and then as a butterfly over the R lanes (group_sum), whatever the
// chunks are: a token's arithmetic does not know where a step was cut.  In memory a head's state is [vdim][dim], so
// that a lane's channels are consecutive and a wave's loads are whole lines.  The next token's inputs are
// read from LDS into registers while this token's sums run.
#define RULE_THREADS 256

template <int R, int DR>
struct RuleShape {
  static constexpr int DMAX = DR * R;                            // key channels this instance holds
  static constexpr int TC = 2048 / DMAX < 16 ? 2048 / DMAX : 16; // tokens a chunk
  static constexpr int CB = 4 * 64 / R;                          // value columns a workgroup
  static constexpr int BUF = (TC * (3 * DMAX + CB + 1) + 3) / 4 * 4;   // floats of one LDS buffer: k, q, g, v, beta
  static constexpr int NI = (TC * DMAX + RULE_THREADS - 1) / RULE_THREADS;
  static constexpr int NV = (TC * CB + RULE_THREADS - 1) / RULE_THREADS;
};

//
// DELTA false is the same walk without the correction: S <- diag(g) S + k v^T; o = S^T q (gated linear attention); beta is
// not read, q is multiplied by q_scale as it is brought in, and the inputs may be elements (IN).  HEAD_DECAY: `decay` holds
// one decay a head [H] that takes the place of the decays per token and channel.
template <int R, int DR, bool DELTA, typename IN, bool HEAD_DECAY = false>
__global__ __launch_bounds__(RULE_THREADS) void delta_rule_kernel(float* __restrict__ out, const IN* __restrict__ qkv, int64_t ld, int q_col,
                                                                  int k_col, int v_col, const float* __restrict__ decay,
                                                                  const elem_t* __restrict__ b, int64_t ldb, float* state, int64_t state_stride,
                                                                  const int32_t* __restrict__ cu_q, const int32_t* __restrict__ positions,
                                                                  const int32_t* __restrict__ slots, int H, int G, int d, int dv, float q_scale) {
  using Sh = RuleShape<R, DR>;
  constexpr int DMAX = Sh::DMAX, TC = Sh::TC, CB = Sh::CB;
  __shared__ __attribute__((aligned(16))) float smem[2 * Sh::BUF];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane % R;
  const int col_in_block = wave * (64 / R) + lane / R;
  const int col = blockIdx.z * CB + col_in_block;
  const bool col_ok = col < dv;
  const int g = h / (H / G);
  const int first = cu_q[s], n = cu_q[s + 1] - first;
  const bool fresh = positions[first] == 0;
  float* S_mem = state + (int64_t)slots[s] * state_stride + ((int64_t)h * dv + (col_ok ? col : 0)) * d + r * DR;
  const bool rows_vec = d % 4 == 0 && (((uintptr_t)S_mem) & 15) == 0;
  float S[DR];
#pragma unroll
  for (int i = 0; i < DR; ++i) S[i] = 0.f;
  if (!fresh && col_ok) {
    if (rows_vec) {
#pragma unroll
      for (int i = 0; i < DR; i += 4) {
        if (r * DR + i < d) {
          const f32x4 v4 = *reinterpret_cast<const f32x4*>(S_mem + i);
          S[i] = v4.x; S[i + 1] = v4.y; S[i + 2] = v4.z; S[i + 3] = v4.w;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < DR; ++i)
        if (r * DR + i < d) S[i] = S_mem[i];
    }
  }

  // What this thread brings in of a chunk: elements e = tid, tid + 256, ... of the chunk's [TC][DMAX] tiles of k, q and
  // the decays, and of its [TC][CB] tile of v; beta by the first TC threads.  Channels beyond d read as k = q = 0, g = 1.
  float pk[Sh::NI], pq[Sh::NI], pg[Sh::NI], pv[Sh::NV], pb = 0.f;
  const float head_g = HEAD_DECAY ? decay[h] : 1.f;
  auto fetch = [&](int chunk) {
    const int t0 = chunk * TC;
#pragma unroll
    for (int it = 0; it < Sh::NI; ++it) {
      const int e = tid + it * RULE_THREADS;
      const int tok = e / DMAX, c = e - tok * DMAX;
      const bool ok = e < TC * DMAX && t0 + tok < n && c < d;
      const int64_t t = first + t0 + (ok ? tok : 0);
      const int cc = ok ? c : 0;
      const float kv = to_f32(qkv[t * ld + k_col + (int64_t)g * d + cc]), qv = to_f32(qkv[t * ld + q_col + (int64_t)g * d + cc]);
      // One decay a head for all tokens and channels (decay [H]), or one per token and channel (decay [T, H, d]).
      const float gv = HEAD_DECAY ? head_g : decay[(t * H + h) * d + cc];
      pk[it] = ok ? kv : 0.f;
      pq[it] = ok ? (DELTA ? qv : qv * q_scale) : 0.f;
      pg[it] = ok ? gv : 1.f;
    }
#pragma unroll
    for (int it = 0; it < Sh::NV; ++it) {
      const int e = tid + it * RULE_THREADS;
      const int tok = e / CB, c = e - tok * CB;
      const bool ok = e < TC * CB && t0 + tok < n && blockIdx.z * CB + c < dv;
      const int64_t t = first + t0 + (ok ? tok : 0);
      const float vv = to_f32(qkv[t * ld + v_col + (int64_t)h * dv + (ok ? blockIdx.z * CB + c : 0)]);
      pv[it] = ok ? vv : 0.f;
    }
    if (DELTA && tid < TC) {
      const bool ok = t0 + tid < n;
      const float bb = to_f32(b[(int64_t)(first + t0 + (ok ? tid : 0)) * ldb + h]);
      pb = ok ? sigmoid_f(bb) : 0.f;
    }
  };
  auto stage = [&](int buffer) {
    float* base = smem + buffer * Sh::BUF;
#pragma unroll
    for (int it = 0; it < Sh::NI; ++it) {
      const int e = tid + it * RULE_THREADS;
      if (e < TC * DMAX) {
        base[e] = pk[it];
        base[TC * DMAX + e] = pq[it];
        base[2 * TC * DMAX + e] = pg[it];
      }
    }
#pragma unroll
    for (int it = 0; it < Sh::NV; ++it) {
      const int e = tid + it * RULE_THREADS;
      if (e < TC * CB) base[3 * TC * DMAX + e] = pv[it];
    }
    if (tid < TC) base[3 * TC * DMAX + TC * CB + tid] = pb;
  };

  const int chunks = (n + TC - 1) / TC;
  fetch(0);
  stage(0);
  __syncthreads();
  for (int chunk = 0; chunk < chunks; ++chunk) {
    const float* base = smem + (chunk & 1) * Sh::BUF;
    if (chunk + 1 < chunks) fetch(chunk + 1);
    const int here = min(TC, n - chunk * TC);
    // The inputs of token `tok` as this lane needs them; asked for one token ahead.
    float kn[DR], qn[DR], gn[DR], vn, bn;
    auto read = [&](int tok) {
      const float* kr = base + tok * DMAX + r * DR;
      const float* qr = kr + TC * DMAX;
      const float* gr = qr + TC * DMAX;
#pragma unroll
      for (int i = 0; i < DR; i += 4) {
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(kr + i), g4 = *reinterpret_cast<const f32x4*>(gr + i);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(qr + i);
        kn[i] = k4.x; kn[i + 1] = k4.y; kn[i + 2] = k4.z; kn[i + 3] = k4.w;
        qn[i] = q4.x; qn[i + 1] = q4.y; qn[i + 2] = q4.z; qn[i + 3] = q4.w;
        gn[i] = g4.x; gn[i + 1] = g4.y; gn[i + 2] = g4.z; gn[i + 3] = g4.w;
      }
      vn = base[3 * TC * DMAX + tok * CB + col_in_block];
      bn = base[3 * TC * DMAX + TC * CB + tok];
    };
    read(0);
    for (int tok = 0; tok < here; ++tok) {
      float kk[DR], qq[DR];
      float dot = 0.f;
      const float v = vn, beta = bn;
#pragma unroll
      for (int i = 0; i < DR; ++i) {
        kk[i] = kn[i];
        qq[i] = qn[i];
        S[i] = S[i] * gn[i];
      }
      if (tok + 1 < here) read(tok + 1);
      // Fused multiply-adds, written out: one instruction and one rounding a step.
      if (DELTA) {
#pragma unroll
        for (int i = 0; i < DR; ++i) dot = __builtin_fmaf(S[i], kk[i], dot);
        dot = group_sum<R>(dot);
      }
      const float u = DELTA ? beta * (v - dot) : v;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DR; ++i) {
        S[i] = __builtin_fmaf(kk[i], u, S[i]);
        o = __builtin_fmaf(S[i], qq[i], o);
      }
      o = group_sum<R>(o);
      if (col_ok && r == 0) out[((int64_t)(first + chunk * TC + tok) * H + h) * dv + col] = o;
    }
    if (chunk + 1 < chunks) stage((chunk + 1) & 1);
    __syncthreads();
  }
  if (col_ok) {
    if (rows_vec) {
#pragma unroll
      for (int i = 0; i < DR; i += 4)
        if (r * DR + i < d) *reinterpret_cast<f32x4*>(S_mem + i) = f32x4{S[i], S[i + 1], S[i + 2], S[i + 3]};
    } else {
#pragma unroll
      for (int i = 0; i < DR; ++i)
        if (r * DR + i < d) S_mem[i] = S[i];
    }
  }
}

// y[t, h, :] = o / sqrt(mean(o^2) + eps) * w * sigmoid(gate[t, h, :]) (gate_kind 1: * silu(gate[t, h, :])), stored as elements in rows of length ldy; the
// columns beyond the heads are set to zero (a projection with padded columns reads them).  One wave per (token, head).
__global__ __launch_bounds__(64) void delta_out_kernel(elem_t* __restrict__ y, int64_t ldy, const float* __restrict__ o,
                                                       const elem_t* __restrict__ gate, int64_t ldg, const void* __restrict__ w, int w_is_f32,
                                                       int H, int dv, float eps, int gate_kind) {
  const int t = blockIdx.x / H, h = blockIdx.x - t * H;
  const float* row = o + ((int64_t)t * H + h) * dv;
  float part = 0.f;
  for (int c = threadIdx.x; c < dv; c += 64) part = part + row[c] * row[c];
  const float rr = rsqrtf(wave_sum_xor(part) / (float)dv + eps);
  for (int c = threadIdx.x; c < dv; c += 64) {
    const float gz = to_f32(gate[(int64_t)t * ldg + (int64_t)h * dv + c]);
    const float gt = gate_kind == 0 ? sigmoid_f(gz) : silu_f(gz);
    y[(int64_t)t * ldy + (int64_t)h * dv + c] = from_f32<elem_t>(((row[c] * rr) * load_weight(w, w_is_f32, c)) * gt);
  }
  if (h == H - 1)
    for (int64_t c = (int64_t)H * dv + threadIdx.x; c < ldy; c += 64) y[(int64_t)t * ldy + c] = from_f32<elem_t>(0.f);
}

// y[t, :] = o[t, :] / sqrt(mean(o[t, :]^2) + eps) * w * sigmoid(gate[t, :]) (gate_kind 1: * silu) over rows of n entries: one
// norm for all heads of a read-out.  One workgroup a row; thread t owns the groups of four entries t, t + 256, ... (n in
// whole groups; a single entry a thread otherwise), sums their squares in that order, a butterfly over the wave follows and
// the four waves' sums are added in wave order.  The columns of y beyond n are set to zero.
template <int V>
__global__ __launch_bounds__(256) void gated_row_norm_kernel(elem_t* __restrict__ y, int64_t ldy, const float* __restrict__ o,
                                                             const elem_t* __restrict__ gate, int64_t ldg, const void* __restrict__ w, int w_is_f32,
                                                             int n, float eps, int gate_kind) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* row = o + (int64_t)t * n;
  float part = 0.f;
  for (int c = threadIdx.x * V; c < n; c += 256 * V) {
#pragma unroll
    for (int j = 0; j < V; ++j) part = part + row[c + j] * row[c + j];
  }
  part = wave_sum_xor(part);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
  __syncthreads();
  const float rr = rsqrtf((((red[0] + red[1]) + red[2]) + red[3]) / (float)n + eps);
  for (int c = threadIdx.x * V; c < n; c += 256 * V) {
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float gz = to_f32(gate[(int64_t)t * ldg + c + j]);
      y[(int64_t)t * ldy + c + j] = from_f32<elem_t>(((row[c + j] * rr) * load_weight(w, w_is_f32, c + j)) * (gate_kind == 0 ? sigmoid_f(gz) : silu_f(gz)));
    }
  }
  for (int64_t c = n + threadIdx.x; c < ldy; c += 256) y[(int64_t)t * ldy + c] = from_f32<elem_t>(0.f);
}

// x[t, col0 : col0 + n] <- silu(x[t, col0 : col0 + n]) in place, in 32-bit, stored as elements: the activation of a projection
// whose outputs feed a recurrence.  A thread takes a 16-byte vector where rows and columns are whole vectors (vec).
__global__ __launch_bounds__(256) void silu_columns_kernel(elem_t* x, int64_t ld, int64_t col0, int n, int T, int vec) {
  const int per = vec ? n / VK_VEC : n;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)T * per) return;
  const int64_t t = i / per;
  const int c = (int)(i - t * per);
  if (vec) {
    float v[VK_VEC];
    elem_t* p = x + t * ld + col0 + (int64_t)c * VK_VEC;
    load_elems(p, v);
#pragma unroll
    for (int j = 0; j < VK_VEC; ++j) v[j] = silu_f(v[j]);
    store_elems(p, v);
  } else {
    elem_t* p = x + t * ld + col0 + c;
    *p = from_f32<elem_t>(silu_f(to_f32(*p)));
  }
}

extern "C" {

// Key channels a lane holds, and lanes that share a value column, for key size d.
static int rule_channels_per_lane(int d) { return d <= 256 ? 4 : (d <= 512 ? 8 : 16); }
int vk_delta_lanes_per_column(int d) {
  int R = 1;
  while (R < 64 && R * rule_channels_per_lane(d) < d) R *= 2;
  return R;
}

// y [T, C] floats from the columns x[:, 0:C] of rows of length ldx; then the tails are moved on.  bias: [C] or null, what
// every channel's sum starts from.
static int conv_launch(float* y, const elem_t* x, int64_t ldx, const elem_t* taps, const elem_t* bias, float* state, int64_t state_stride,
                       int64_t tail_offset, const int32_t* token_seq, const int32_t* cu_q, const int32_t* positions, const int32_t* slots, int T,
                       int S, int C, int K, hipStream_t st) {
  VK_REQUIRE(T >= 0 && S >= 0 && C > 0 && K >= 1 && K <= DELTA_MAX_TAPS + 1, "short convolution: bad sizes T=%d C=%d taps=%d (at most %d)", T, C, K,
             DELTA_MAX_TAPS + 1);
  VK_REQUIRE(ldx >= C && tail_offset >= 0 && state_stride >= tail_offset + (int64_t)(K - 1) * C, "short convolution: the state does not hold the tails");
  if (T == 0 || S == 0) return 0;
  const int by = (C + 255) / 256 < 64 ? (C + 255) / 256 : 64;
  delta_conv_kernel<<<dim3(T, by), 256, 0, st>>>(y, x, ldx, taps, state, state_stride, tail_offset, token_seq, cu_q, positions, slots, C, K, bias);
  if (vk_check_launch("short convolution")) return 1;
  if (K > 1) {
    delta_conv_tail_kernel<<<dim3(S, by), 256, 0, st>>>(x, ldx, state, state_stride, tail_offset, cu_q, positions, slots, C, K);
    return vk_check_launch("short convolution (tails)");
  }
  return 0;
}

int vk_delta_conv(float* y, const elem_t* x, int64_t ldx, const elem_t* taps, float* state, int64_t state_stride, int64_t tail_offset,
                  const int32_t* token_seq, const int32_t* cu_q, const int32_t* positions, const int32_t* slots, int T, int S, int C, int K,
                  hipStream_t st) {
  return conv_launch(y, x, ldx, taps, nullptr, state, state_stride, tail_offset, token_seq, cu_q, positions, slots, T, S, C, K, st);
}

// The same with a bias per channel.
int vk_delta_conv_bias(float* y, const elem_t* x, int64_t ldx, const elem_t* taps, const elem_t* bias, float* state, int64_t state_stride,
                       int64_t tail_offset, const int32_t* token_seq, const int32_t* cu_q, const int32_t* positions, const int32_t* slots, int T,
                       int S, int C, int K, hipStream_t st) {
  VK_REQUIRE(bias != nullptr, "short convolution: the bias is missing");
  return conv_launch(y, x, ldx, taps, bias, state, state_stride, tail_offset, token_seq, cu_q, positions, slots, T, S, C, K, st);
}

int vk_delta_unit(float* x, int64_t ld, int col0, int T, int heads, int d, float eps, float scale, hipStream_t st) {
  VK_REQUIRE(T >= 0 && heads > 0 && d > 0 && ld >= col0 + (int64_t)heads * d, "unit norm: bad sizes");
  if (T == 0) return 0;
  VK_REQUIRE((int64_t)T * heads < (1ll << 31), "unit norm: too many rows");
  delta_unit_kernel<<<T * heads, 64, 0, st>>>(x, ld, col0, heads, d, eps, scale);
  return vk_check_launch("unit norm");
}

int vk_delta_decay(float* g, const elem_t* a, const void* dt_bias, const void* A_log, int w_is_f32, int T, int H, int d, hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && d > 0, "decay: bad sizes");
  const int64_t numel = (int64_t)T * H * d;
  if (numel == 0) return 0;
  delta_decay_kernel<<<(unsigned)((numel + 255) / 256), 256, 0, st>>>(g, a, dt_bias, A_log, w_is_f32, d, H * d, numel);
  return vk_check_launch("decay");
}

// x[:, q_col ..] (G heads of d) and x[:, k_col ..] become unit vectors (q times q_scale); g [T, H, d] = the decays of a [T, H d].
int vk_delta_prep(float* x, int64_t ld, int q_col, int k_col, int T, int G, int H, int d, float unit_eps, float q_scale, float* g,
                  const elem_t* a, const void* dt_bias, const void* A_log, int w_is_f32, hipStream_t st) {
  VK_REQUIRE(T >= 0 && G > 0 && H > 0 && d > 0 && ld >= (int64_t)G * d + (q_col > k_col ? q_col : k_col), "delta prep: bad sizes");
  if (T == 0) return 0;
  VK_REQUIRE((int64_t)T * (2 * G + H) < (1ll << 31), "delta prep: too many rows");
  delta_prep_kernel<<<T * (2 * G + H), 64, 0, st>>>(x, ld, q_col, k_col, G, H, d, unit_eps, q_scale, g, a, dt_bias, A_log, w_is_f32);
  return vk_check_launch("delta prep");
}

// out [T, H, dv] floats.  qkv: float rows of length ld with q (G heads of d) at q_col, k at k_col, v (H heads of dv) at
// v_col; decay [T, H, d] floats; b: elements, beta's pre-activation of head h at b[t * ldb + h].  state: per slot,
// the H states at its start, each [dv][d].
extern "C++" {
template <bool DELTA, typename IN, bool HEAD_DECAY = false>
static int rule_launch(float* out, const IN* qkv, int64_t ld, int q_col, int k_col, int v_col, const float* decay, const elem_t* b, int64_t ldb,
                       float* state, int64_t state_stride, const int32_t* cu_q, const int32_t* positions, const int32_t* slots, int S, int H, int G,
                       int d, int dv, float q_scale, hipStream_t st) {
  VK_REQUIRE(S >= 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0, "delta rule: bad sizes H=%d G=%d d=%d dv=%d", H, G, d, dv);
  VK_REQUIRE(decay != nullptr, "delta rule: the decays are missing");
  VK_REQUIRE(d <= 1024, "delta rule: key size %d exceeds 1024", d);
  VK_REQUIRE(state_stride >= (int64_t)H * d * dv, "delta rule: the state is too small");
  if (S == 0) return 0;
  const int R = vk_delta_lanes_per_column(d), DR = rule_channels_per_lane(d);
  const int cols = 4 * 64 / R;
  const dim3 grid(S, H, (dv + cols - 1) / cols);
  VK_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "delta rule: too many heads or columns");
#define RULE(RR, DD) \
  delta_rule_kernel<RR, DD, DELTA, IN, HEAD_DECAY><<<grid, RULE_THREADS, 0, st>>>(out, qkv, ld, q_col, k_col, v_col, decay, b, ldb, state, state_stride, cu_q, positions, slots, H, G, d, dv, q_scale)
  if (DR == 4) {
    switch (R) {
      case 1: RULE(1, 4); break;
      case 2: RULE(2, 4); break;
      case 4: RULE(4, 4); break;
      case 8: RULE(8, 4); break;
      case 16: RULE(16, 4); break;
      case 32: RULE(32, 4); break;
      default: RULE(64, 4); break;
    }
  } else if (DR == 8) {
    RULE(64, 8);
  } else {
    RULE(64, 16);
  }
#undef RULE
  return vk_check_launch("delta rule");
}
}  // extern "C++"

int vk_delta_rule(float* out, const float* qkv, int64_t ld, int q_col, int k_col, int v_col, const float* decay, const elem_t* b, int64_t ldb,
                  float* state, int64_t state_stride, const int32_t* cu_q, const int32_t* positions, const int32_t* slots, int S, int H, int G,
                  int d, int dv, hipStream_t st) {
  return rule_launch<true, float>(out, qkv, ld, q_col, k_col, v_col, decay, b, ldb, state, state_stride, cu_q, positions, slots, S, H, G, d, dv, 1.f,
                                  st);
}

// Gated linear attention: g [T, H, d] = sigmoid(a + bias)^(1 / root) = exp(-softplus(-(a + bias)) / root) from the
// elements a (rows of length lda) and the bias [H d], in 32-bit.
int vk_gla_decay(float* g, const elem_t* a, int64_t lda, const void* bias, int w_is_f32, int T, int HD, float root, hipStream_t st) {
  VK_REQUIRE(T >= 0 && HD > 0 && lda >= HD && root > 0.f, "linear attention decay: bad sizes T=%d channels=%d root=%g", T, HD, (double)root);
  const int64_t numel = (int64_t)T * HD;
  if (numel == 0) return 0;
  gla_decay_kernel<<<(unsigned)((numel + 255) / 256), 256, 0, st>>>(g, a, lda, bias, w_is_f32, HD, 1.f / root, numel);
  return vk_check_launch("linear attention decay");
}

// The recurrence S <- diag(g) S + k v^T, o = S^T (q * q_scale) per head.  x: element rows of length ld with q (H heads of
// d) at q_col, k at k_col, v (H heads of dv) at v_col; decay [T, H, d] floats; out [T, H, dv] floats; state as vk_delta_rule's.
int vk_gla_rule(float* out, const elem_t* x, int64_t ld, int q_col, int k_col, int v_col, const float* decay, float* state, int64_t state_stride,
                const int32_t* cu_q, const int32_t* positions, const int32_t* slots, int S, int H, int d, int dv, float q_scale, hipStream_t st) {
  return rule_launch<false, elem_t>(out, x, ld, q_col, k_col, v_col, decay, nullptr, 0, state, state_stride, cu_q, positions, slots, S, H, H, d, dv,
                                    q_scale, st);
}

// Linear attention with one fixed decay a head: S <- decay[h] S + k v^T, o = S^T (q * q_scale), with q, k (H heads of d) and v
// (H heads of dv) the elements at the three columns of x.  head_decay [H] floats.
int vk_linear_rule(float* out, const elem_t* x, int64_t ld, int q_col, int k_col, int v_col, const float* head_decay, float* state,
                   int64_t state_stride, const int32_t* cu_q, const int32_t* positions, const int32_t* slots, int S, int H, int d, int dv, float q_scale,
                   hipStream_t st) {
  VK_REQUIRE(head_decay != nullptr, "linear attention: the heads' decays are missing");
  return rule_launch<false, elem_t, true>(out, x, ld, q_col, k_col, v_col, head_decay, nullptr, 0, state, state_stride, cu_q, positions, slots, S, H, H, d,
                                          dv, q_scale, st);
}

// y [T, ldy] elements from o [T, n] floats, gate rows of length ldg and w [n]: gated_row_norm_kernel.
int vk_gated_row_norm(elem_t* y, int64_t ldy, const float* o, const elem_t* gate, int64_t ldg, const void* w, int w_is_f32, int T, int n, float eps,
                      int gate_kind, hipStream_t st) {
  VK_REQUIRE(T >= 0 && n > 0 && ldg >= n && ldy >= n && (gate_kind == 0 || gate_kind == 1), "gated row norm: bad sizes T=%d n=%d", T, n);
  if (T == 0) return 0;
  if (n % 4 == 0) gated_row_norm_kernel<4><<<T, 256, 0, st>>>(y, ldy, o, gate, ldg, w, w_is_f32, n, eps, gate_kind);
  else gated_row_norm_kernel<1><<<T, 256, 0, st>>>(y, ldy, o, gate, ldg, w, w_is_f32, n, eps, gate_kind);
  return vk_check_launch("gated row norm");
}

// silu in place on the columns [col0, col0 + n) of x [T, ld].
int vk_silu_columns(elem_t* x, int64_t ld, int64_t col0, int n, int T, hipStream_t st) {
  VK_REQUIRE(T >= 0 && n > 0 && col0 >= 0 && ld >= col0 + n, "silu of columns: bad sizes T=%d n=%d", T, n);
  if (T == 0) return 0;
  const int vec = n % VK_VEC == 0 && ld % VK_VEC == 0 && col0 % VK_VEC == 0 && (uintptr_t)x % 16 == 0;
  const int64_t total = (int64_t)T * (vec ? n / VK_VEC : n);
  silu_columns_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>(x, ld, col0, n, T, vec);
  return vk_check_launch("silu of columns");
}

int vk_delta_out(elem_t* y, int64_t ldy, const float* o, const elem_t* gate, int64_t ldg, const void* w, int w_is_f32, int T, int H, int dv,
                 float eps, hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && dv > 0 && ldg >= (int64_t)H * dv && ldy >= (int64_t)H * dv, "delta read-out: bad sizes");
  if (T == 0) return 0;
  VK_REQUIRE((int64_t)T * H < (1ll << 31), "delta read-out: too many rows");
  delta_out_kernel<<<T * H, 64, 0, st>>>(y, ldy, o, gate, ldg, w, w_is_f32, H, dv, eps, 0);
  return vk_check_launch("delta read-out");
}

// The same read-out with a choice of gate: gate_kind 0 is the logistic function of the gate's input, 1 is z * logistic(z).
int vk_gated_head_norm(elem_t* y, int64_t ldy, const float* o, const elem_t* gate, int64_t ldg, const void* w, int w_is_f32, int T, int H, int dv,
                       float eps, int gate_kind, hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && dv > 0 && ldg >= (int64_t)H * dv && ldy >= (int64_t)H * dv && (gate_kind == 0 || gate_kind == 1),
             "gated head norm: bad sizes");
  if (T == 0) return 0;
  VK_REQUIRE((int64_t)T * H < (1ll << 31), "gated head norm: too many rows");
  delta_out_kernel<<<T * H, 64, 0, st>>>(y, ldy, o, gate, ldg, w, w_is_f32, H, dv, eps, gate_kind);
  return vk_check_launch("gated head norm");
}

}  // extern "C"
