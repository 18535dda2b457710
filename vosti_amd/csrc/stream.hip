// Kernels for a residual stream that is kept in 32-bit whatever the element type: the embedding with sinusoidal
// positions added, the norm that reads the stream and writes elements, the norm of a sublayer's output that is
// scaled and added to the stream, the weighted sum of the stream's earlier states, a row gather, and the cap of
// the logits.
//
// Norms here are y = x * rsqrt(mean(x^2) + eps) * (offset + w): offset 1 is the weight stored around zero, offset 0
// the plain weight.  One workgroup per row; thread t owns the elements t, t + 256, ... of the row, its partial sum
// runs over them in that order, a wave butterfly follows and the four wave sums are added in wave order, so the
// order depends on the row's length alone.
#include "common.h"
#include "vec.h"

#define STREAM_THREADS 256

__device__ __forceinline__ float stream_block_sum(float v, float* red) {
  v = wave_sum_xor(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = red[0];
  s = s + red[1];
  s = s + red[2];
  s = s + red[3];
  return s;
}

// out[t, 2i] = table[id, 2i] + sin(p * f[i]); out[t, 2i + 1] = table[id, 2i + 1] + cos(p * f[i]); angles in 32-bit.
__global__ __launch_bounds__(STREAM_THREADS) void embed_sinusoid_kernel(float* __restrict__ out, const elem_t* __restrict__ table,
                                                                        const int32_t* __restrict__ ids,
                                                                        const int32_t* __restrict__ positions,
                                                                        const float* __restrict__ inv_freq, int H) {
  const int t = blockIdx.x;
  const elem_t* src = table + (int64_t)ids[t] * H;
  const float p = (float)positions[t];
  float* dst = out + (int64_t)t * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    const float angle = p * inv_freq[c >> 1];
    dst[c] = to_f32(src[c]) + ((c & 1) ? cosf(angle) : sinf(angle));
  }
}

template <bool IN_F32>
__device__ __forceinline__ float stream_load(const void* x, int64_t i) {
  return IN_F32 ? static_cast<const float*>(x)[i] : to_f32(static_cast<const elem_t*>(x)[i]);
}

// out (elements) = norm of a row of the stream (IN_F32) or of elements.
template <bool IN_F32>
__global__ __launch_bounds__(STREAM_THREADS) void stream_norm_kernel(elem_t* __restrict__ out, const void* __restrict__ x,
                                                                     const void* __restrict__ w, int w_is_f32, int H, float eps,
                                                                     float offset) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * H;
  float part = 0.f;
  for (int c = threadIdx.x; c < H; c += STREAM_THREADS) {
    const float v = stream_load<IN_F32>(x, base + c);
    part = part + v * v;
  }
  const float rr = rsqrtf(stream_block_sum(part, red) / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += STREAM_THREADS) {
    const float v = stream_load<IN_F32>(x, base + c);
    out[base + c] = from_f32<elem_t>((v * rr) * (offset + load_weight(w, w_is_f32, c)));
  }
}

// out = base + mult * norm(y), rows of the stream; out may be base.
template <typename Y>     // the normed rows: elements, or floats
__global__ __launch_bounds__(STREAM_THREADS) void stream_norm_add_kernel(float* out, const float* base_rows, const Y* __restrict__ y,
                                                                         const void* __restrict__ w, int w_is_f32, int H, float eps,
                                                                         float offset, float mult, elem_t* __restrict__ rounded) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * H;
  float part = 0.f;
  for (int c = threadIdx.x; c < H; c += STREAM_THREADS) {
    const float v = to_f32(y[base + c]);
    part = part + v * v;
  }
  const float rr = rsqrtf(stream_block_sum(part, red) / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += STREAM_THREADS) {
    const float v = to_f32(y[base + c]);
    const float n = (v * rr) * (offset + load_weight(w, w_is_f32, c));
    const float o = base_rows[base + c] + mult * n;
    out[base + c] = o;
    if (rounded != nullptr) rounded[base + c] = from_f32<elem_t>(o);      // the new stream as the next sublayer reads it
  }
}

// The same two norms for rows of whole 16-byte vectors that fit a workgroup's registers: thread t owns the vectors t,
// t + 256, ... (NV of them at most), reads them once, and sums their squares element by element in that order.
template <bool IN_F32, int NV>
__global__ __launch_bounds__(STREAM_THREADS) void stream_norm_vec_kernel(elem_t* __restrict__ out, const void* __restrict__ x,
                                                                         const void* __restrict__ w, int w_is_f32, int H, float eps,
                                                                         float offset) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * H;
  const int nvec = H / 4;
  f32x4 v[NV];
  float part = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = threadIdx.x + j * STREAM_THREADS;
    v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < nvec) {
      if (IN_F32) {
        v[j] = *reinterpret_cast<const f32x4*>(static_cast<const float*>(x) + base + 4 * c);
      } else {
        const elem_t* p = static_cast<const elem_t*>(x) + base + 4 * c;
        v[j] = f32x4{to_f32(p[0]), to_f32(p[1]), to_f32(p[2]), to_f32(p[3])};
      }
    }
    part = part + v[j].x * v[j].x;
    part = part + v[j].y * v[j].y;
    part = part + v[j].z * v[j].z;
    part = part + v[j].w * v[j].w;
  }
  const float rr = rsqrtf(stream_block_sum(part, red) / (float)H + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = threadIdx.x + j * STREAM_THREADS;
    if (c < nvec) {
      elem_t* o = out + base + 4 * c;
      o[0] = from_f32<elem_t>((v[j].x * rr) * (offset + load_weight(w, w_is_f32, 4 * c)));
      o[1] = from_f32<elem_t>((v[j].y * rr) * (offset + load_weight(w, w_is_f32, 4 * c + 1)));
      o[2] = from_f32<elem_t>((v[j].z * rr) * (offset + load_weight(w, w_is_f32, 4 * c + 2)));
      o[3] = from_f32<elem_t>((v[j].w * rr) * (offset + load_weight(w, w_is_f32, 4 * c + 3)));
    }
  }
}

template <int NV, typename Y>
__global__ __launch_bounds__(STREAM_THREADS) void stream_norm_add_vec_kernel(float* out, const float* base_rows, const Y* __restrict__ y,
                                                                             const void* __restrict__ w, int w_is_f32, int H, float eps,
                                                                             float offset, float mult, elem_t* __restrict__ rounded) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * H;
  const int nvec = H / 4;
  f32x4 v[NV], b[NV];
  float part = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = threadIdx.x + j * STREAM_THREADS;
    v[j] = b[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < nvec) {
      const Y* p = y + base + 4 * c;
      v[j] = f32x4{to_f32(p[0]), to_f32(p[1]), to_f32(p[2]), to_f32(p[3])};
      b[j] = *reinterpret_cast<const f32x4*>(base_rows + base + 4 * c);
    }
    part = part + v[j].x * v[j].x;
    part = part + v[j].y * v[j].y;
    part = part + v[j].z * v[j].z;
    part = part + v[j].w * v[j].w;
  }
  const float rr = rsqrtf(stream_block_sum(part, red) / (float)H + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = threadIdx.x + j * STREAM_THREADS;
    if (c < nvec) {
      f32x4 o;
      o.x = b[j].x + mult * ((v[j].x * rr) * (offset + load_weight(w, w_is_f32, 4 * c)));
      o.y = b[j].y + mult * ((v[j].y * rr) * (offset + load_weight(w, w_is_f32, 4 * c + 1)));
      o.z = b[j].z + mult * ((v[j].z * rr) * (offset + load_weight(w, w_is_f32, 4 * c + 2)));
      o.w = b[j].w + mult * ((v[j].w * rr) * (offset + load_weight(w, w_is_f32, 4 * c + 3)));
      *reinterpret_cast<f32x4*>(out + base + 4 * c) = o;
      if (rounded != nullptr) {
        elem_t* r = rounded + base + 4 * c;
        r[0] = from_f32<elem_t>(o.x); r[1] = from_f32<elem_t>(o.y); r[2] = from_f32<elem_t>(o.z); r[3] = from_f32<elem_t>(o.w);
      }
    }
  }
}

// out[e] = sum over j < n of coef[j] * states[j * stride + e], added in ascending j from zero.
__global__ __launch_bounds__(256) void stream_mix_kernel(float* __restrict__ out, const float* __restrict__ states, int64_t stride,
                                                         const void* __restrict__ coef, int coef_is_f32, int n, int64_t numel) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= numel) return;
  float acc = 0.f;
  for (int j = 0; j < n; ++j) acc = acc + load_weight(coef, coef_is_f32, j) * states[j * stride + e];
  out[e] = acc;
}

// The same, four consecutive elements a thread (numel and stride multiples of 4, 16-byte aligned).
__global__ __launch_bounds__(256) void stream_mix_vec_kernel(f32x4* __restrict__ out, const f32x4* __restrict__ states, int64_t stride4,
                                                             const void* __restrict__ coef, int coef_is_f32, int n, int64_t numel4) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= numel4) return;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < n; ++j) {
    const float cj = load_weight(coef, coef_is_f32, j);
    const f32x4 v = states[j * stride4 + e];
    acc.x = acc.x + cj * v.x;
    acc.y = acc.y + cj * v.y;
    acc.z = acc.z + cj * v.z;
    acc.w = acc.w + cj * v.w;
  }
  out[e] = acc;
}

__global__ __launch_bounds__(256) void gather_rows_f32_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                              const int32_t* __restrict__ rows, int H) {
  const float* src = x + (int64_t)rows[blockIdx.x] * H;
  float* dst = out + (int64_t)blockIdx.x * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) dst[c] = src[c];
}

// x <- cap * tanh(x / cap), in 32-bit, stored as elements.
__global__ __launch_bounds__(256) void softcap_kernel(elem_t* x, float cap, int64_t n) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e < n) x[e] = from_f32<elem_t>(cap * tanhf(to_f32(x[e]) / cap));
}

// out[t, :] = table[ids[t], :] * scale, as floats: the residual stream of a model whose embedding is multiplied by a constant.
__global__ __launch_bounds__(STREAM_THREADS) void embed_scaled_kernel(float* __restrict__ out, const elem_t* __restrict__ table,
                                                                      const int32_t* __restrict__ ids, int H, float scale) {
  const elem_t* src = table + (int64_t)ids[blockIdx.x] * H;
  float* dst = out + (int64_t)blockIdx.x * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) dst[c] = to_f32(src[c]) * scale;
}

// out = base + (a + b) (b may be null: out = base + a), element by element; a and b are floats or elements.
__global__ __launch_bounds__(256) void stream_add_kernel(float* out, const float* base, const void* __restrict__ a, int a_is_f32,
                                                         const void* __restrict__ b, int b_is_f32, int64_t n) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  float v = a_is_f32 ? static_cast<const float*>(a)[e] : to_f32(static_cast<const elem_t*>(a)[e]);
  if (b != nullptr) v = v + (b_is_f32 ? static_cast<const float*>(b)[e] : to_f32(static_cast<const elem_t*>(b)[e]));
  out[e] = base[e] + v;
}

// out = ca * norm_a(a) + cb * norm_b(b), rows of floats: each input row divided by its own root mean square and
// multiplied by its own weight.  One workgroup per row, sums in stream_block_sum's order.
__global__ __launch_bounds__(STREAM_THREADS) void stream_pair_norm_kernel(float* __restrict__ out, const elem_t* __restrict__ a,
                                                                          const void* __restrict__ wa, const elem_t* __restrict__ b,
                                                                          const void* __restrict__ wb, int w_is_f32, int H, float eps, float ca,
                                                                          float cb) {
  __shared__ float red_a[4], red_b[4];
  const int64_t base = (int64_t)blockIdx.x * H;
  float pa = 0.f, pb = 0.f;
  for (int c = threadIdx.x; c < H; c += STREAM_THREADS) {
    const float va = to_f32(a[base + c]), vb = to_f32(b[base + c]);
    pa = pa + va * va;
    pb = pb + vb * vb;
  }
  const float ra = rsqrtf(stream_block_sum(pa, red_a) / (float)H + eps);
  const float rb = rsqrtf(stream_block_sum(pb, red_b) / (float)H + eps);
  for (int c = threadIdx.x; c < H; c += STREAM_THREADS) {
    const float na = (to_f32(a[base + c]) * ra) * load_weight(wa, w_is_f32, c);
    const float nb = (to_f32(b[base + c]) * rb) * load_weight(wb, w_is_f32, c);
    out[base + c] = ca * na + cb * nb;
  }
}

// The same for rows of whole 16-byte vectors that fit a workgroup's registers (thread t owns the vectors t, t + 256, ...).
template <int NV>
__global__ __launch_bounds__(STREAM_THREADS) void stream_pair_norm_vec_kernel(float* __restrict__ out, const elem_t* __restrict__ a,
                                                                              const void* __restrict__ wa, const elem_t* __restrict__ b,
                                                                              const void* __restrict__ wb, int w_is_f32, int H, float eps,
                                                                              float ca, float cb) {
  __shared__ float red_a[4], red_b[4];
  const int64_t base = (int64_t)blockIdx.x * H;
  const int nvec = H / 4;
  f32x4 va[NV], vb[NV];
  float pa = 0.f, pb = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = threadIdx.x + j * STREAM_THREADS;
    va[j] = vb[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < nvec) {
      const elem_t *p = a + base + 4 * c, *q = b + base + 4 * c;
      va[j] = f32x4{to_f32(p[0]), to_f32(p[1]), to_f32(p[2]), to_f32(p[3])};
      vb[j] = f32x4{to_f32(q[0]), to_f32(q[1]), to_f32(q[2]), to_f32(q[3])};
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      pa = pa + va[j][e] * va[j][e];
      pb = pb + vb[j][e] * vb[j][e];
    }
  }
  const float ra = rsqrtf(stream_block_sum(pa, red_a) / (float)H + eps);
  const float rb = rsqrtf(stream_block_sum(pb, red_b) / (float)H + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = threadIdx.x + j * STREAM_THREADS;
    if (c < nvec) {
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o[e] = ca * ((va[j][e] * ra) * load_weight(wa, w_is_f32, 4 * c + e)) + cb * ((vb[j][e] * rb) * load_weight(wb, w_is_f32, 4 * c + e));
      *reinterpret_cast<f32x4*>(out + base + 4 * c) = o;
    }
  }
}

// out[t, c] = gelu(gate[t, c]) * table[ids[t], first + c] for c < n, zero for n <= c < ldo: a token's slice of a second
// embedding table, gated by a projection of the stream.  gelu(z) = z / 2 * (1 + tanh(sqrt(2 / pi) * (z + 0.044715 z^3))), in 32-bit.
__global__ __launch_bounds__(256) void side_gate_kernel(elem_t* __restrict__ out, int64_t ldo, const elem_t* __restrict__ gate, int64_t ldg,
                                                        const elem_t* __restrict__ table, int64_t table_width, const int32_t* __restrict__ ids, int first,
                                                        int n, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / ldo;
  const int c = (int)(i - t * ldo);
  float v = 0.f;
  if (c < n) {
    const float z = to_f32(gate[t * ldg + c]);
    const float inner = 0.7978845608028654f * (z + 0.044715f * ((z * z) * z));
    v = ((0.5f * z) * (1.f + tanhf(inner))) * to_f32(table[(int64_t)ids[t] * table_width + first + c]);
  }
  out[i] = from_f32<elem_t>(v);
}

extern "C" {

int vk_embed_sinusoid(float* out, const elem_t* table, const int32_t* ids, const int32_t* positions, const float* inv_freq, int T,
                      int H, int V, hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && H % 2 == 0 && V > 0, "sinusoidal embedding: bad sizes T=%d H=%d V=%d (the width must be even)", T, H, V);
  if (T == 0) return 0;
  embed_sinusoid_kernel<<<T, STREAM_THREADS, 0, st>>>(out, table, ids, positions, inv_freq, H);
  return vk_check_launch("sinusoidal embedding");
}

// x: rows of floats (x_is_f32) or of elements; out: elements.
int vk_stream_norm(elem_t* out, const void* x, int x_is_f32, const void* w, int w_is_f32, int rows, int H, float eps, float offset,
                   hipStream_t st) {
  VK_REQUIRE(rows >= 0 && H > 0 && eps >= 0.f, "stream norm: bad sizes rows=%d H=%d", rows, H);
  if (rows == 0) return 0;
  const int nv = (H / 4 + STREAM_THREADS - 1) / STREAM_THREADS;
  if (H % 4 == 0 && nv <= 8 && (uintptr_t)x % 16 == 0) {
#define NORM_VEC(F32, NV) stream_norm_vec_kernel<F32, NV><<<rows, STREAM_THREADS, 0, st>>>(out, x, w, w_is_f32, H, eps, offset)
    if (x_is_f32) { if (nv <= 1) NORM_VEC(true, 1); else if (nv <= 2) NORM_VEC(true, 2); else if (nv <= 4) NORM_VEC(true, 4); else NORM_VEC(true, 8); }
    else { if (nv <= 1) NORM_VEC(false, 1); else if (nv <= 2) NORM_VEC(false, 2); else if (nv <= 4) NORM_VEC(false, 4); else NORM_VEC(false, 8); }
#undef NORM_VEC
  } else if (x_is_f32) {
    stream_norm_kernel<true><<<rows, STREAM_THREADS, 0, st>>>(out, x, w, w_is_f32, H, eps, offset);
  } else {
    stream_norm_kernel<false><<<rows, STREAM_THREADS, 0, st>>>(out, x, w, w_is_f32, H, eps, offset);
  }
  return vk_check_launch("stream norm");
}

extern "C++" {
template <typename Y>
static int norm_add_launch(float* out, const float* base, const Y* y, const void* w, int w_is_f32, int rows, int H, float eps, float offset, float mult,
                           hipStream_t st, elem_t* rounded = nullptr) {
  VK_REQUIRE(rows >= 0 && H > 0 && eps >= 0.f, "stream norm-add: bad sizes rows=%d H=%d", rows, H);
  if (rows == 0) return 0;
  const int nv = (H / 4 + STREAM_THREADS - 1) / STREAM_THREADS;
  if (H % 4 == 0 && nv <= 8 && (uintptr_t)out % 16 == 0 && (uintptr_t)base % 16 == 0) {
#define NORM_ADD_VEC(NV) stream_norm_add_vec_kernel<NV, Y><<<rows, STREAM_THREADS, 0, st>>>(out, base, y, w, w_is_f32, H, eps, offset, mult, rounded)
    if (nv <= 1) NORM_ADD_VEC(1); else if (nv <= 2) NORM_ADD_VEC(2); else if (nv <= 4) NORM_ADD_VEC(4); else NORM_ADD_VEC(8);
#undef NORM_ADD_VEC
  } else {
    stream_norm_add_kernel<Y><<<rows, STREAM_THREADS, 0, st>>>(out, base, y, w, w_is_f32, H, eps, offset, mult, rounded);
  }
  return vk_check_launch("stream norm-add");
}
}  // extern "C++"

int vk_stream_norm_add(float* out, const float* base, const elem_t* y, const void* w, int w_is_f32, int rows, int H, float eps,
                       float offset, float mult, hipStream_t st) {
  return norm_add_launch<elem_t>(out, base, y, w, w_is_f32, rows, H, eps, offset, mult, st);
}

// The same for rows that a sublayer left in 32-bit.
int vk_stream_norm_add_f32(float* out, const float* base, const float* y, const void* w, int w_is_f32, int rows, int H, float eps,
                           float offset, float mult, hipStream_t st) {
  return norm_add_launch<float>(out, base, y, w, w_is_f32, rows, H, eps, offset, mult, st);
}

// The same two, and the new rows of the stream rounded to elements as well (rounded [rows, H]): what a sublayer that reads
// the stream as it is takes next, without a launch of its own.
int vk_stream_norm_add_rounded(float* out, const float* base, const elem_t* y, const void* w, int w_is_f32, int rows, int H, float eps, float offset,
                               float mult, elem_t* rounded, hipStream_t st) {
  VK_REQUIRE(rounded != nullptr, "stream norm-add: the rounded rows have no memory");
  return norm_add_launch<elem_t>(out, base, y, w, w_is_f32, rows, H, eps, offset, mult, st, rounded);
}
int vk_stream_norm_add_f32_rounded(float* out, const float* base, const float* y, const void* w, int w_is_f32, int rows, int H, float eps, float offset,
                                   float mult, elem_t* rounded, hipStream_t st) {
  VK_REQUIRE(rounded != nullptr, "stream norm-add: the rounded rows have no memory");
  return norm_add_launch<float>(out, base, y, w, w_is_f32, rows, H, eps, offset, mult, st, rounded);
}

int vk_stream_mix(float* out, const float* states, int64_t stride, const void* coef, int coef_is_f32, int n, int64_t numel,
                  hipStream_t st) {
  VK_REQUIRE(n > 0 && numel >= 0 && stride >= numel, "stream mix: bad sizes n=%d numel=%lld stride=%lld", n, (long long)numel, (long long)stride);
  if (numel == 0) return 0;
  if (numel % 4 == 0 && stride % 4 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)states % 16 == 0)
    stream_mix_vec_kernel<<<(unsigned)((numel / 4 + 255) / 256), 256, 0, st>>>(reinterpret_cast<f32x4*>(out), reinterpret_cast<const f32x4*>(states),
                                                                              stride / 4, coef, coef_is_f32, n, numel / 4);
  else
    stream_mix_kernel<<<(unsigned)((numel + 255) / 256), 256, 0, st>>>(out, states, stride, coef, coef_is_f32, n, numel);
  return vk_check_launch("stream mix");
}

int vk_gather_rows_f32(float* out, const float* x, const int32_t* rows, int R, int H, hipStream_t st) {
  VK_REQUIRE(R >= 0 && H > 0, "gather_rows: bad sizes R=%d H=%d", R, H);
  if (R == 0) return 0;
  gather_rows_f32_kernel<<<R, 256, 0, st>>>(out, x, rows, H);
  return vk_check_launch("gather_rows (32-bit)");
}

int vk_softcap(elem_t* x, float cap, int64_t n, hipStream_t st) {
  VK_REQUIRE(cap > 0.f && n >= 0, "softcap: the cap must be positive");
  if (n == 0) return 0;
  softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(x, cap, n);
  return vk_check_launch("softcap");
}

int vk_embed_scaled(float* out, const elem_t* table, const int32_t* ids, int T, int H, int V, float scale, hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && V > 0, "scaled embedding: bad sizes T=%d H=%d V=%d", T, H, V);
  if (T == 0) return 0;
  embed_scaled_kernel<<<T, STREAM_THREADS, 0, st>>>(out, table, ids, H, scale);
  return vk_check_launch("scaled embedding");
}

int vk_stream_add(float* out, const float* base, const void* a, int a_is_f32, const void* b, int b_is_f32, int64_t n, hipStream_t st) {
  VK_REQUIRE(n >= 0 && a != nullptr, "stream add: bad sizes");
  if (n == 0) return 0;
  stream_add_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(out, base, a, a_is_f32, b, b_is_f32, n);
  return vk_check_launch("stream add");
}

int vk_stream_pair_norm(float* out, const elem_t* a, const void* wa, const elem_t* b, const void* wb, int w_is_f32, int rows, int H, float eps,
                        float ca, float cb, hipStream_t st) {
  VK_REQUIRE(rows >= 0 && H > 0 && eps >= 0.f, "pair norm: bad sizes rows=%d H=%d", rows, H);
  if (rows == 0) return 0;
  const int nv = (H / 4 + STREAM_THREADS - 1) / STREAM_THREADS;
  if (H % 4 == 0 && nv <= 8 && (uintptr_t)out % 16 == 0) {
#define PAIR_VEC(NV) stream_pair_norm_vec_kernel<NV><<<rows, STREAM_THREADS, 0, st>>>(out, a, wa, b, wb, w_is_f32, H, eps, ca, cb)
    if (nv <= 1) PAIR_VEC(1); else if (nv <= 2) PAIR_VEC(2); else if (nv <= 4) PAIR_VEC(4); else PAIR_VEC(8);
#undef PAIR_VEC
  } else {
    stream_pair_norm_kernel<<<rows, STREAM_THREADS, 0, st>>>(out, a, wa, b, wb, w_is_f32, H, eps, ca, cb);
  }
  return vk_check_launch("pair norm");
}

// out [T, ldo] elements from gate [T, ldg] (its first n columns) and the columns [first, first + n) of table [V, table_width]
// at the rows ids name; the columns of out beyond n are zero.  Ids must lie below V: the caller checks them on the host.
int vk_side_gate(elem_t* out, int64_t ldo, const elem_t* gate, int64_t ldg, const elem_t* table, int64_t table_width, const int32_t* ids, int first,
                 int n, int T, hipStream_t st) {
  VK_REQUIRE(T >= 0 && n > 0 && first >= 0 && ldo >= n && ldg >= n && table_width >= (int64_t)first + n, "token side input: bad sizes n=%d first=%d", n, first);
  if (T == 0) return 0;
  const int64_t total = (int64_t)T * ldo;
  side_gate_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>(out, ldo, gate, ldg, table, table_width, ids, first, n, total);
  return vk_check_launch("token side input");
}

}  // extern "C"
