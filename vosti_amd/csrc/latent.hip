// Attention through a latent: what stands between its projections and the paged attention kernels.
//
// A token keeps one row for all heads: the normed latent c (r entries), then the part of the key that is rotated by the
// position (dr entries), then zeros up to the cache's head size D.  The same row without the rotated part is the token's
// value.  A head's query meets it as [W_uk[h]^T q_flat | rotate(q_rot) | 0]: the score (q_flat . W_uk[h] c + q_rot . k_rot)
// is one dot product of D entries, every head reads the one cached row (one kv head), and a head's output is W_uv[h] times
// the weighted sum of the cached latents.  So the cache holds r + dr numbers a token whatever the number of heads.
//
//   vk_norm_columns   y = x[:, col : col + n] / sqrt(mean(.^2) + eps) * w as elements, in rows padded with zeros
//   vk_gemm_heads     one product a head: out[t, h, :] = W[h] x[t, h, :]
//   vk_latent_post    norm of the latent, rotation of the key part and of every head's rotated query part, cache store
#include "common.h"
#include "mma.h"
#include "vec.h"

// One workgroup a row: y[t, 0:n] = norm(x[t, col : col + n]) * w, y[t, n:ldy] = 0.  The sum of squares runs over a thread's
// elements t, t + 256, ... in order, then as a butterfly over a wave, and the four waves' sums are added in wave order: the
// order depends on n alone.
__global__ __launch_bounds__(256) void norm_columns_kernel(elem_t* __restrict__ y, int64_t ldy, const elem_t* __restrict__ x, int64_t ldx, int col,
                                                           int n, const void* __restrict__ w, int w_is_f32, float eps) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const elem_t* row = x + (int64_t)t * ldx + col;
  float part = 0.f;
  for (int c = threadIdx.x; c < n; c += 256) {
    const float v = to_f32(row[c]);
    part = part + v * v;
  }
  part = wave_sum_xor(part);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
  __syncthreads();
  const float rr = rsqrtf((((red[0] + red[1]) + red[2]) + red[3]) / (float)n + eps);
  for (int c = threadIdx.x; c < ldy; c += 256)
    y[(int64_t)t * ldy + c] = from_f32<elem_t>(c < n ? (to_f32(row[c]) * rr) * load_weight(w, w_is_f32, c) : 0.f);
}

// out[t, h * os + f] = sum over k < K of w[h][f][k] * x[t, h * xs + k] for f < N: a product a head, its weights [H, N, K].
// A wave takes 16 rows and 64 output features of one head (four accumulators that share the rows' fragments); a workgroup's
// four waves take four such row tiles side by side, so that they read the same weights.  The sums have the order of this
// library's other products: the reduction axis in chunks of 512 elements, a chunk's products added from zero over ascending
// slabs of 64 bytes with the weights as first operand, the chunk sums added to a zero total in chunk order.
#define HEADS_KC 512
__global__ __launch_bounds__(256) void gemm_heads_kernel(elem_t* __restrict__ out, int64_t ldo, int64_t os, const elem_t* __restrict__ x, int64_t ldx,
                                                         int64_t xs, const elem_t* __restrict__ w, int T, int N, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kq = lane >> 4;
  const int f0 = blockIdx.x * 64, t0 = (blockIdx.y * 4 + wave) * 16, h = blockIdx.z;
  if (t0 >= T) return;
  const bool x_ok = t0 + r16 < T;
  const elem_t* xr = x + (int64_t)(x_ok ? t0 + r16 : 0) * ldx + (int64_t)h * xs + kq * VK_VEC;
  const elem_t* wr[4];
  bool w_ok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    w_ok[j] = f0 + 16 * j + r16 < N;
    wr[j] = w + ((int64_t)h * N + (w_ok[j] ? f0 + 16 * j + r16 : 0)) * K + kq * VK_VEC;
  }
  f32x4 total[4], acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) total[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int c0 = 0; c0 < K; c0 += HEADS_KC) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int end = min(K, c0 + HEADS_KC);
#pragma unroll 2
    for (int k = c0; k < end; k += VK_SLAB) {
      const bool k_ok = k + kq * VK_VEC < K;
      const frag_t fx = load_frag(xr + k, x_ok && k_ok);
      frag_t fw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) fw[j] = load_frag(wr[j] + k, w_ok[j] && k_ok);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = mma_slab(fw[j], fx, acc[j]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      total[j].x = total[j].x + acc[j].x; total[j].y = total[j].y + acc[j].y; total[j].z = total[j].z + acc[j].z; total[j].w = total[j].w + acc[j].w;
    }
  }
  // Lane l holds features f0 + 16 j + 4 * (l / 16) + i of row l % 16.
  if (!x_ok) return;
  elem_t* o = out + (int64_t)(t0 + r16) * ldo + (int64_t)h * os;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int f = f0 + 16 * j + kq * 4 + i;
      if (f < N) o[f] = from_f32<elem_t>(total[j][i]);
    }
  }
}

struct LatentPostArgs {
  const elem_t* kv;       // [T, ldkv]: the latent before its norm (r entries), then the key part to rotate (dr); null: queries only
  int64_t ldkv;
  const elem_t* q;        // [T, ldq]: head h's part to rotate at columns [h * qs + q_first, .. + dr)
  int64_t ldq, qs;
  int q_first;
  elem_t* q_out;          // [T, H, D]: the rotated part goes to columns [r, r + dr), zeros behind it
  elem_t* kc;             // [pages, 1, P, D]
  elem_t* vc;             // [pages, 1, D, P]
  const void* w;          // [r] the latent's norm weight
  int w_is_f32;
  const float* inv_freq;  // [dr / 2]
  const int32_t* positions;
  const int32_t* slots;   // page * P + offset, or -1
  int H, r, dr, D, P, neighbours;
  float eps;
};

// Element j of a part of dr entries after its rotation: pair c is the entries 2c and 2c + 1 (neighbours) or c and c + dr/2.
__device__ __forceinline__ float rotated_entry(const elem_t* part, int j, int dr, int neighbours, float posf, const float* __restrict__ inv_freq) {
  const int half = dr / 2;
  const int pair = neighbours ? j >> 1 : (j < half ? j : j - half);
  const bool second = neighbours ? (j & 1) != 0 : j >= half;
  const int other = neighbours ? (j ^ 1) : (second ? j - half : j + half);
  const float angle = posf * inv_freq[pair];
  const float cs = cosf(angle), sn = sinf(angle);
  const float mine = to_f32(part[j]), theirs = to_f32(part[other]);
  return second ? mine * cs + theirs * sn : mine * cs - theirs * sn;
}

// One workgroup a token.  Queries: every head's rotated part and the zeros behind it.  Keys and values (where the layer has
// a latent of its own and the token a slot): c = norm(latent) rounded to the element type, the key row [c | rotated part |
// 0], the value column [c | 0].
__global__ __launch_bounds__(256) void latent_post_kernel(LatentPostArgs a) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const float posf = (float)a.positions[t];
  const int tail = a.D - a.r;
  for (int i = tid; i < a.H * tail; i += 256) {
    const int h = i / tail, j = i - h * tail;
    const elem_t* part = a.q + (int64_t)t * a.ldq + (int64_t)h * a.qs + a.q_first;
    const float v = j < a.dr ? rotated_entry(part, j, a.dr, a.neighbours, posf, a.inv_freq) : 0.f;
    a.q_out[((int64_t)t * a.H + h) * a.D + a.r + j] = from_f32<elem_t>(v);
  }
  if (a.kv == nullptr) return;
  const int slot = a.slots[t];
  if (slot < 0) return;
  const elem_t* row = a.kv + (int64_t)t * a.ldkv;
  // Every wave sums the row's squares for itself, in the one order.
  float part = 0.f;
  for (int c = tid & 63; c < a.r; c += 64) {
    const float v = to_f32(row[c]);
    part = part + v * v;
  }
  const float rr = rsqrtf(wave_sum_xor(part) / (float)a.r + a.eps);
  const int page = slot / a.P, off = slot - page * a.P;
  elem_t* krow = a.kc + ((int64_t)page * a.P + off) * a.D;
  elem_t* vcol = a.vc + (int64_t)page * a.D * a.P + off;
  for (int c = tid; c < a.D; c += 256) {
    float kval, vval;
    if (c < a.r) {
      kval = vval = (to_f32(row[c]) * rr) * load_weight(a.w, a.w_is_f32, c);
    } else {
      kval = c < a.r + a.dr ? rotated_entry(row + a.r, c - a.r, a.dr, a.neighbours, posf, a.inv_freq) : 0.f;
      vval = 0.f;
    }
    krow[c] = from_f32<elem_t>(kval);
    vcol[(int64_t)c * a.P] = from_f32<elem_t>(vval);
  }
}

extern "C" {

int vk_norm_columns(elem_t* y, int64_t ldy, const elem_t* x, int64_t ldx, int col, int n, const void* w, int w_is_f32, float eps, int T,
                    hipStream_t st) {
  VK_REQUIRE(T >= 0 && n > 0 && col >= 0 && ldx >= (int64_t)col + n && ldy >= n, "norm of columns: bad sizes T=%d n=%d col=%d", T, n, col);
  if (T == 0) return 0;
  norm_columns_kernel<<<T, 256, 0, st>>>(y, ldy, x, ldx, col, n, w, w_is_f32, eps);
  return vk_check_launch("norm of columns");
}

// out rows of length ldo with head h's N outputs from column h * os; x rows of length ldx with head h's K inputs from
// column h * xs; w [H, N, K].  K in whole 16-byte vectors, as are both strides of x and the operands' addresses.
int vk_gemm_heads(elem_t* out, int64_t ldo, int64_t os, const elem_t* x, int64_t ldx, int64_t xs, const elem_t* w, int T, int H, int N, int K,
                  hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && N > 0 && K > 0 && K % VK_VEC == 0 && ldx % VK_VEC == 0 && xs % VK_VEC == 0,
             "product a head: bad sizes H=%d N=%d K=%d (K and the input's strides in whole 16-byte vectors)", H, N, K);
  VK_REQUIRE(ldx >= (int64_t)(H - 1) * xs + K && ldo >= (int64_t)(H - 1) * os + N && os >= 0 && xs >= 0, "product a head: the rows do not hold the heads");
  VK_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "product a head: operands must be 16-byte aligned");
  VK_REQUIRE(H <= 65535 && (T + 63) / 64 <= 65535, "product a head: too many heads or rows for one launch");
  if (T == 0) return 0;
  gemm_heads_kernel<<<dim3((N + 63) / 64, (T + 63) / 64, H), 256, 0, st>>>(out, ldo, os, x, ldx, xs, w, T, N, K);
  return vk_check_launch("product a head");
}

// kv null: the layer reads another's cache, and only the queries are written.
int vk_latent_post(const elem_t* kv, int64_t ldkv, const elem_t* q, int64_t ldq, int64_t qs, int q_first, elem_t* q_out, elem_t* kc, elem_t* vc,
                   const void* w, int w_is_f32, float eps, const float* inv_freq, int neighbours, const int32_t* positions, const int32_t* slots, int T,
                   int H, int r, int dr, int D, int P, hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && r > 0 && dr > 0 && dr % 2 == 0 && D >= r + dr, "latent attention: bad sizes H=%d r=%d dr=%d D=%d", H, r, dr, D);
  VK_REQUIRE(q != nullptr && q_out != nullptr && inv_freq != nullptr && positions != nullptr && qs >= q_first + dr && ldq >= (int64_t)(H - 1) * qs + q_first + dr,
             "latent attention: the queries' rows do not hold the heads");
  VK_REQUIRE(kv == nullptr || (ldkv >= r + dr && kc != nullptr && vc != nullptr && w != nullptr && slots != nullptr && P > 0),
             "latent attention: a store needs the caches, the norm's weight and slots");
  VK_REQUIRE(neighbours == 0 || neighbours == 1, "latent attention: 'neighbours' is 0 or 1");
  if (T == 0) return 0;
  LatentPostArgs a;
  a.kv = kv; a.ldkv = ldkv; a.q = q; a.ldq = ldq; a.qs = qs; a.q_first = q_first; a.q_out = q_out; a.kc = kc; a.vc = vc; a.w = w; a.w_is_f32 = w_is_f32;
  a.inv_freq = inv_freq; a.positions = positions; a.slots = slots; a.H = H; a.r = r; a.dr = dr; a.D = D; a.P = P; a.neighbours = neighbours; a.eps = eps;
  latent_post_kernel<<<T, 256, 0, st>>>(a);
  return vk_check_launch("latent attention");
}

}  // extern "C"
