// Layer-norm flavoured ops around an f32 residual stream, and the row norms of
// the recurrent mixers.
//
//   layer_norm_stream        out = (x - mean) / sqrt(var + eps) * w   (no bias)
//   stream_add_layer_norm    x += LN(sa * a + sb * b) * w * ls, optionally also
//                            next_out = LN(x) * next_w of the updated row
//   stream_add_vec           x += other + vec (vec broadcast over rows)
//   gated_group_norm         RMS norm of an f32 row in equal parts with a gate:
//                            silu(gate) before the norm or sigmoid(gate) after
//   qk_norm_cache_write      per-head RMS norm of queries and keys, query
//                            temperature by position, keys and values stored
//                            in the paged cache
//
// The two stream norms keep the row in registers when the width is a multiple
// of 4 and at most 256 * 4 * 8 (16-byte accesses, every input read once); other
// widths take the any-width kernels, which re-read the row from L1/L2.
//
// All are memory-bound row kernels: one workgroup per row (or per row part),
// statistics in f32 with the variance taken as the mean of squared deviations
// from the mean (second pass over the row, which sits in L1/L2 by then).  Each
// thread touches the same columns in every pass, so a row that is updated in
// place needs no barrier between the update and the pass that reads it back.

#include "common.h"

namespace {

// every reduction of a kernel gets its own scratch: block_reduce_sum leaves
// its result in scratch[0], which a following reduction would overwrite while
// slower waves still read it
DEVINLINE float reduce_sum(float x, float* scratch) { return block_reduce_sum(x, scratch); }

template <typename T>
__global__ __launch_bounds__(256) void layer_norm_stream_kernel(
    T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
    float eps, int width) {
  __shared__ float r0[16], r1[16];
  const long row = blockIdx.x;
  const float* xr = x + row * width;
  float s = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) s += xr[c];
  const float mu = reduce_sum(s, r0) / width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float d = xr[c] - mu;
    ss += d * d;
  }
  const float inv = 1.0f / sqrtf(reduce_sum(ss, r1) / width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    out[row * width + c] = ScalarOps<T>::from_f32((xr[c] - mu) * inv * w[c]);
}

template <typename T>
__global__ __launch_bounds__(256) void stream_add_layer_norm_kernel(
    float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b,
    float sa, float sb, const float* __restrict__ w, const float* __restrict__ ls,
    float eps, int width, T* __restrict__ next_out, const float* __restrict__ next_w,
    float next_eps) {
  __shared__ float r0[16], r1[16], r2[16], r3[16];
  const long row = blockIdx.x;
  float* xr = x + row * width;
  const T* ar = a + row * width;
  const T* br = b ? b + row * width : nullptr;
  auto y_at = [&](int c) {
    float y = sa * ScalarOps<T>::to_f32(ar[c]);
    if (br) y += sb * ScalarOps<T>::to_f32(br[c]);
    return y;
  };
  float s = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) s += y_at(c);
  const float mu = reduce_sum(s, r0) / width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float d = y_at(c) - mu;
    ss += d * d;
  }
  const float inv = 1.0f / sqrtf(reduce_sum(ss, r1) / width + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = (y_at(c) - mu) * inv * w[c];
    if (ls) v *= ls[c];
    const float nx = xr[c] + v;
    xr[c] = nx;
    s2 += nx;
  }
  if (next_out == nullptr) return;
  const float mu2 = reduce_sum(s2, r2) / width;
  float ss2 = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float d = xr[c] - mu2;
    ss2 += d * d;
  }
  const float inv2 = 1.0f / sqrtf(reduce_sum(ss2, r3) / width + next_eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    next_out[row * width + c] = ScalarOps<T>::from_f32((xr[c] - mu2) * inv2 * next_w[c]);
}

// ---- register-cached variants: width % 4 == 0, width <= 1024 * NCH ---------

template <typename T> DEVINLINE float4 ld4(const T* p);
template <> DEVINLINE float4 ld4<float>(const float* p) {
  return *reinterpret_cast<const float4*>(p);
}
template <> DEVINLINE float4 ld4<__hip_bfloat16>(const __hip_bfloat16* p) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(t.x << 16), __uint_as_float(t.x & 0xffff0000u),
                     __uint_as_float(t.y << 16), __uint_as_float(t.y & 0xffff0000u));
}
template <typename T> DEVINLINE void st4(T* p, float4 v);
template <> DEVINLINE void st4<float>(float* p, float4 v) {
  *reinterpret_cast<float4*>(p) = v;
}
template <> DEVINLINE void st4<__hip_bfloat16>(__hip_bfloat16* p, float4 v) {
  union { __hip_bfloat16 h[4]; uint2 u; } o;
  o.h[0] = __float2bfloat16(v.x); o.h[1] = __float2bfloat16(v.y);
  o.h[2] = __float2bfloat16(v.z); o.h[3] = __float2bfloat16(v.w);
  *reinterpret_cast<uint2*>(p) = o.u;
}

// mean and 1/sqrt(var + eps) of the row held in v[NCH] (chunks past the width
// are zero and masked out of the deviations)
template <int NCH>
DEVINLINE void row_stats(const float4* v, int width, float eps, float* r_a, float* r_b,
                         float& mu, float& inv) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
  mu = reduce_sum(s, r_a) / width;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    if ((int)(threadIdx.x * 4 + i * 1024) < width) {
      const float a = v[i].x - mu, b = v[i].y - mu, c = v[i].z - mu, d = v[i].w - mu;
      ss += (a * a + b * b) + (c * c + d * d);
    }
  }
  inv = 1.0f / sqrtf(reduce_sum(ss, r_b) / width + eps);
}

template <typename T, int NCH>
__global__ __launch_bounds__(256) void layer_norm_stream_reg_kernel(
    T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
    float eps, int width) {
  __shared__ float r0[16], r1[16];
  const long row = blockIdx.x;
  float4 v[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x * 4 + i * 1024;
    v[i] = c < width ? ld4<float>(x + row * width + c) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float mu, inv;
  row_stats<NCH>(v, width, eps, r0, r1, mu, inv);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x * 4 + i * 1024;
    if (c < width) {
      const float4 ww = ld4<float>(w + c);
      st4<T>(out + row * width + c,
             make_float4((v[i].x - mu) * inv * ww.x, (v[i].y - mu) * inv * ww.y,
                         (v[i].z - mu) * inv * ww.z, (v[i].w - mu) * inv * ww.w));
    }
  }
}

template <typename T, int NCH>
__global__ __launch_bounds__(256) void stream_add_layer_norm_reg_kernel(
    float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b,
    float sa, float sb, const float* __restrict__ w, const float* __restrict__ ls,
    float eps, int width, T* __restrict__ next_out, const float* __restrict__ next_w,
    float next_eps) {
  __shared__ float r0[16], r1[16], r2[16], r3[16];
  const long row = blockIdx.x;
  float4 v[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x * 4 + i * 1024;
    v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < width) {
      const float4 t = ld4<T>(a + row * width + c);
      v[i] = make_float4(sa * t.x, sa * t.y, sa * t.z, sa * t.w);
      if (b != nullptr) {
        const float4 u = ld4<T>(b + row * width + c);
        v[i].x += sb * u.x; v[i].y += sb * u.y; v[i].z += sb * u.z; v[i].w += sb * u.w;
      }
    }
  }
  float mu, inv;
  row_stats<NCH>(v, width, eps, r0, r1, mu, inv);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x * 4 + i * 1024;
    if (c < width) {
      float4 g = ld4<float>(w + c);
      if (ls != nullptr) {
        const float4 l = ld4<float>(ls + c);
        g.x *= l.x; g.y *= l.y; g.z *= l.z; g.w *= l.w;
      }
      const float4 xo = ld4<float>(x + row * width + c);
      v[i] = make_float4(xo.x + (v[i].x - mu) * inv * g.x, xo.y + (v[i].y - mu) * inv * g.y,
                         xo.z + (v[i].z - mu) * inv * g.z, xo.w + (v[i].w - mu) * inv * g.w);
      st4<float>(x + row * width + c, v[i]);
    }
  }
  if (next_out == nullptr) return;
  float mu2, inv2;
  row_stats<NCH>(v, width, next_eps, r2, r3, mu2, inv2);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x * 4 + i * 1024;
    if (c < width) {
      const float4 ww = ld4<float>(next_w + c);
      st4<T>(next_out + row * width + c,
             make_float4((v[i].x - mu2) * inv2 * ww.x, (v[i].y - mu2) * inv2 * ww.y,
                         (v[i].z - mu2) * inv2 * ww.z, (v[i].w - mu2) * inv2 * ww.w));
    }
  }
}

__global__ void stream_add_vec_kernel(float* __restrict__ x, const float* __restrict__ other,
                                      const float* __restrict__ vec, int width, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    float v = x[i] + vec[i % width];
    if (other) v += other[i];
    x[i] = v;
  }
}

// grid (rows, groups); y [rows, C] f32, gate rows strided
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ gate,
    long gate_stride, const float* __restrict__ w, float eps, int cols, int gsize,
    int gate_first) {
  __shared__ float r0[16];
  const long row = blockIdx.x;
  const int c0 = blockIdx.y * gsize;
  const float* yr = y + row * cols + c0;
  const T* gr = gate + row * gate_stride + c0;
  float ss = 0.f;
  for (int c = threadIdx.x; c < gsize; c += blockDim.x) {
    float v = yr[c];
    if (gate_first) {
      const float g = ScalarOps<T>::to_f32(gr[c]);
      v *= g / (1.0f + expf(-g));
    }
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(reduce_sum(ss, r0) / gsize + eps);
  for (int c = threadIdx.x; c < gsize; c += blockDim.x) {
    const float g = ScalarOps<T>::to_f32(gr[c]);
    const float sg = 1.0f / (1.0f + expf(-g));
    float v = yr[c];
    if (gate_first) v = v * (g * sg) * inv * w[c0 + c];
    else v = v * inv * w[c0 + c] * sg;
    out[row * cols + c0 + c] = ScalarOps<T>::from_f32(v);
  }
}

// One wave per (token, unit): units 0..H-1 are query heads, H..H+G-1 key
// heads, H+G..H+2G-1 value heads.  grid (tokens, ceil(units / 4)), 256 threads.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_cache_write_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long q_st,
    const T* __restrict__ k, long k_st, const T* __restrict__ v, long v_st,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const long* __restrict__ positions, float temp_coef, int temp_every,
    T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slot_mapping, int heads, int kv_heads, int dim,
    int vdim) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int unit = blockIdx.y * (blockDim.x / WAVE_SIZE) + threadIdx.x / WAVE_SIZE;
  if (unit >= heads + 2 * kv_heads) return;
  const long slot = slot_mapping[t];
  if (unit >= heads + kv_heads) {           // value head: copy into the cache
    if (slot < 0) return;
    const int g = unit - heads - kv_heads;
    const T* src = v + t * v_st + (long)g * vdim;
    T* dst = v_cache + (slot * kv_heads + g) * vdim;
    for (int c = lane; c < vdim; c += WAVE_SIZE) dst[c] = src[c];
    return;
  }
  const bool is_q = unit < heads;
  const int hh = is_q ? unit : unit - heads;
  if (!is_q && slot < 0) return;
  const T* src = is_q ? q + t * q_st + (long)hh * dim : k + t * k_st + (long)hh * dim;
  float ss = 0.f;
  for (int c = lane; c < dim; c += WAVE_SIZE) {
    const float x = ScalarOps<T>::to_f32(src[c]);
    ss += x * x;
  }
  ss = wave_reduce_sum(ss);
  float f = 1.0f / sqrtf(ss / dim + eps);
  const float* w = is_q ? qw : kw;
  T* dst;
  if (is_q) {
    if (temp_every > 0) {
      const long p = positions[t];
      f *= 1.0f + temp_coef * logf((float)((p + 1) / temp_every) + 1.0f);
    }
    dst = q_out + (t * heads + hh) * dim;
  } else {
    dst = k_cache + (slot * kv_heads + hh) * dim;
  }
  for (int c = lane; c < dim; c += WAVE_SIZE)
    dst[c] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(src[c]) * f * w[c]);
}

// Vector variant of gated_group_norm: gsize % 4 == 0, the part held in
// registers (gsize <= blockDim * 4 * NCH), every input read once.
template <typename T, int NCH>
__global__ __launch_bounds__(256) void gated_group_norm_reg_kernel(
    T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ gate,
    long gate_stride, const float* __restrict__ w, float eps, int cols, int gsize,
    int gate_first) {
  __shared__ float r0[16];
  const long row = blockIdx.x;
  const int c0 = blockIdx.y * gsize;
  const float* yr = y + row * cols + c0;
  const T* gr = gate + row * gate_stride + c0;
  float4 v[NCH], sg[NCH];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = (threadIdx.x + i * blockDim.x) * 4;
    v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    sg[i] = v[i];
    if (c < gsize) {
      v[i] = ld4<float>(yr + c);
      const float4 g = ld4<T>(gr + c);
      sg[i] = make_float4(1.0f / (1.0f + expf(-g.x)), 1.0f / (1.0f + expf(-g.y)),
                          1.0f / (1.0f + expf(-g.z)), 1.0f / (1.0f + expf(-g.w)));
      if (gate_first) {
        v[i].x *= g.x * sg[i].x; v[i].y *= g.y * sg[i].y;
        v[i].z *= g.z * sg[i].z; v[i].w *= g.w * sg[i].w;
      }
      ss += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
    }
  }
  const float inv = 1.0f / sqrtf(reduce_sum(ss, r0) / gsize + eps);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = (threadIdx.x + i * blockDim.x) * 4;
    if (c < gsize) {
      const float4 ww = ld4<float>(w + c0 + c);
      float4 o = make_float4(v[i].x * inv * ww.x, v[i].y * inv * ww.y,
                             v[i].z * inv * ww.z, v[i].w * inv * ww.w);
      if (!gate_first) { o.x *= sg[i].x; o.y *= sg[i].y; o.z *= sg[i].z; o.w *= sg[i].w; }
      st4<T>(out + row * cols + c0 + c, o);
    }
  }
}

// Vector variant of qk_norm_cache_write: 16 lanes per (token, unit), 16-byte
// accesses; dim, vdim and the row strides are multiples of the vector length.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_cache_write_vec_kernel(
    T* __restrict__ q_out, const T* __restrict__ q, long q_st,
    const T* __restrict__ k, long k_st, const T* __restrict__ v, long v_st,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const long* __restrict__ positions, float temp_coef, int temp_every,
    T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slot_mapping, int heads, int kv_heads, int dim,
    int vdim) {
  constexpr int E = Vec16<T>::kElems;
  constexpr int LPU = 16;
  const long t = blockIdx.x;
  const int lane = threadIdx.x % LPU;
  const int unit = blockIdx.y * (256 / LPU) + threadIdx.x / LPU;
  if (unit >= heads + 2 * kv_heads) return;   // whole 16-lane groups leave together
  const long slot = slot_mapping[t];
  if (unit >= heads + kv_heads) {
    if (slot < 0) return;
    const int g = unit - heads - kv_heads;
    const T* src = v + t * v_st + (long)g * vdim;
    T* dst = v_cache + (slot * kv_heads + g) * vdim;
    for (int c = lane * E; c < vdim; c += LPU * E) store16(dst + c, load16(src + c));
    return;
  }
  const bool is_q = unit < heads;
  const int hh = is_q ? unit : unit - heads;
  if (!is_q && slot < 0) return;
  const T* src = is_q ? q + t * q_st + (long)hh * dim : k + t * k_st + (long)hh * dim;
  float ss = 0.f;
  for (int c = lane * E; c < dim; c += LPU * E) {
    const Vec16<T> x = load16(src + c);
#pragma unroll
    for (int u = 0; u < E; ++u) {
      const float f = ScalarOps<T>::to_f32(x.data[u]);
      ss += f * f;
    }
  }
  ss = group_reduce_sum<LPU>(ss);
  float f = 1.0f / sqrtf(ss / dim + eps);
  const float* w = is_q ? qw : kw;
  T* dst;
  if (is_q) {
    if (temp_every > 0) {
      const long p = positions[t];
      f *= 1.0f + temp_coef * logf((float)((p + 1) / temp_every) + 1.0f);
    }
    dst = q_out + (t * heads + hh) * dim;
  } else {
    dst = k_cache + (slot * kv_heads + hh) * dim;
  }
  for (int c = lane * E; c < dim; c += LPU * E) {
    Vec16<T> x = load16(src + c);
#pragma unroll
    for (int u = 0; u < E; ++u)
      x.data[u] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(x.data[u]) * f * w[c + u]);
    store16(dst + c, x);
  }
}

template <typename P>
inline bool al16(const P* p) {   // 8 bytes are enough for 4 bf16, 16 for 4 f32
  return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0;
}

inline int grid_for(long n, int block) {
  long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

}  // namespace

template <typename T>
void launch_layer_norm_stream(T* out, const float* x, const float* w, float eps,
                              int rows, int width, hipStream_t s) {
  const int nch = (width + 1023) / 1024;
  if (width % 4 == 0 && nch <= 8 && al16(out) && al16(x) && al16(w)) {
    if (nch <= 1) layer_norm_stream_reg_kernel<T, 1><<<rows, 256, 0, s>>>(out, x, w, eps, width);
    else if (nch <= 2) layer_norm_stream_reg_kernel<T, 2><<<rows, 256, 0, s>>>(out, x, w, eps, width);
    else if (nch <= 4) layer_norm_stream_reg_kernel<T, 4><<<rows, 256, 0, s>>>(out, x, w, eps, width);
    else layer_norm_stream_reg_kernel<T, 8><<<rows, 256, 0, s>>>(out, x, w, eps, width);
    return;
  }
  layer_norm_stream_kernel<T><<<rows, 256, 0, s>>>(out, x, w, eps, width);
}

template <typename T>
void launch_stream_add_layer_norm(float* x, const T* a, const T* b, float sa,
                                  float sb, const float* w, const float* ls,
                                  float eps, int rows, int width, T* next_out,
                                  const float* next_w, float next_eps,
                                  hipStream_t s) {
  const int nch = (width + 1023) / 1024;
  if (width % 4 == 0 && nch <= 8 && al16(x) && al16(a) && al16(b) && al16(w) &&
      al16(ls) && al16(next_out) && al16(next_w)) {
#define SALN(N)                                                                \
    stream_add_layer_norm_reg_kernel<T, N><<<rows, 256, 0, s>>>(               \
        x, a, b, sa, sb, w, ls, eps, width, next_out, next_w, next_eps)
    if (nch <= 1) SALN(1);
    else if (nch <= 2) SALN(2);
    else if (nch <= 4) SALN(4);
    else SALN(8);
#undef SALN
    return;
  }
  stream_add_layer_norm_kernel<T><<<rows, 256, 0, s>>>(
      x, a, b, sa, sb, w, ls, eps, width, next_out, next_w, next_eps);
}

void launch_stream_add_vec(float* x, const float* other, const float* vec,
                           int width, long n, hipStream_t s) {
  stream_add_vec_kernel<<<grid_for(n, 256), 256, 0, s>>>(x, other, vec, width, n);
}

template <typename T>
void launch_gated_group_norm(T* out, const float* y, const T* gate,
                             long gate_stride, const float* w, float eps,
                             int rows, int cols, int groups, int gate_first,
                             hipStream_t s) {
  const int gsize = cols / groups;
  dim3 grid(rows, groups);
  if (gsize % 4 == 0 && gate_stride % 4 == 0 && gsize <= 4096 && al16(out) &&
      al16(y) && al16(gate) && al16(w)) {
    const int q4 = gsize / 4;
    const int vb = q4 <= 64 ? 64 : (q4 <= 128 ? 128 : 256);
    if (q4 <= vb)
      gated_group_norm_reg_kernel<T, 1><<<grid, vb, 0, s>>>(out, y, gate, gate_stride, w,
                                                           eps, cols, gsize, gate_first);
    else
      gated_group_norm_reg_kernel<T, 4><<<grid, vb, 0, s>>>(out, y, gate, gate_stride, w,
                                                           eps, cols, gsize, gate_first);
    return;
  }
  const int block = gsize <= 64 ? 64 : (gsize <= 128 ? 128 : 256);
  gated_group_norm_kernel<T><<<grid, block, 0, s>>>(out, y, gate, gate_stride, w, eps,
                                                   cols, gsize, gate_first);
}

template <typename T>
void launch_qk_norm_cache_write(T* q_out, const T* q, long q_st, const T* k,
                                long k_st, const T* v, long v_st, const float* qw,
                                const float* kw, float eps, const long* positions,
                                float temp_coef, int temp_every, T* k_cache,
                                T* v_cache, const long* slot_mapping, int tokens,
                                int heads, int kv_heads, int dim, int vdim,
                                hipStream_t s) {
  const int units = heads + 2 * kv_heads;
  const int e = 16 / sizeof(T);
  if (dim % e == 0 && vdim % e == 0 && q_st % e == 0 && k_st % e == 0 &&
      v_st % e == 0 && al16(q_out) && al16(q) && al16(k) && al16(v) &&
      al16(k_cache) && al16(v_cache)) {
    dim3 vgrid(tokens, (units + 15) / 16);
    qk_norm_cache_write_vec_kernel<T><<<vgrid, 256, 0, s>>>(
        q_out, q, q_st, k, k_st, v, v_st, qw, kw, eps, positions, temp_coef,
        temp_every, k_cache, v_cache, slot_mapping, heads, kv_heads, dim, vdim);
    return;
  }
  dim3 grid(tokens, (units + 3) / 4);
  qk_norm_cache_write_kernel<T><<<grid, 256, 0, s>>>(
      q_out, q, q_st, k, k_st, v, v_st, qw, kw, eps, positions, temp_coef,
      temp_every, k_cache, v_cache, slot_mapping, heads, kv_heads, dim, vdim);
}

#define INSTANTIATE(T)                                                          \
  template void launch_layer_norm_stream<T>(T*, const float*, const float*,     \
                                            float, int, int, hipStream_t);      \
  template void launch_stream_add_layer_norm<T>(                                \
      float*, const T*, const T*, float, float, const float*, const float*,     \
      float, int, int, T*, const float*, float, hipStream_t);                   \
  template void launch_gated_group_norm<T>(T*, const float*, const T*, long,    \
                                           const float*, float, int, int, int,  \
                                           int, hipStream_t);                   \
  template void launch_qk_norm_cache_write<T>(                                  \
      T*, const T*, long, const T*, long, const T*, long, const float*,         \
      const float*, float, const long*, float, int, T*, T*, const long*, int,   \
      int, int, int, int, hipStream_t);
INSTANTIATE(float)
INSTANTIATE(__hip_bfloat16)
