// Ops around an f32 residual stream.
//
// Models that keep their residual in f32 read it through an RMS norm into the
// compute dtype (bf16 or f32), run projections there, and add the results back
// in f32.  All of these are memory-bound row or elementwise kernels: one
// workgroup per row for the norms (sum of squares in f32, block reduce), grid
// stride loops otherwise.  Rotation angles, norm statistics and the stream
// itself never leave f32.

#include "common.h"

DEVINLINE float gelu_tanh_f32(float z) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  return 0.5f * z * (1.0f + tanhf(k * (z + 0.044715f * z * z * z)));
}

// out = gelu_tanh(x) [* mul]; mul rows may be strided (a column slice)
template <typename T>
__global__ void gelu_tanh_kernel(T* __restrict__ out, const T* __restrict__ x,
                                 const T* __restrict__ mul, long mul_stride,
                                 int cols, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    float y = gelu_tanh_f32(ScalarOps<T>::to_f32(x[i]));
    if (mul != nullptr) {
      const long r = i / cols;
      const int c = (int)(i - r * cols);
      y *= ScalarOps<T>::to_f32(mul[r * mul_stride + c]);
    }
    out[i] = ScalarOps<T>::from_f32(y);
  }
}

// out[t, :] = float(table[ids[t], :]) * scale
template <typename T>
__global__ void embedding_scaled_kernel(float* __restrict__ out,
                                        const long* __restrict__ ids,
                                        const T* __restrict__ table,
                                        float scale, int width) {
  const long t = blockIdx.x;
  const T* row = table + ids[t] * (long)width;
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    out[t * width + c] = ScalarOps<T>::to_f32(row[c]) * scale;
}

// out = x / sqrt(mean(x^2) + eps) * (offset + w), x and w f32
template <typename T>
__global__ void rms_norm_stream_kernel(T* __restrict__ out,
                                       const float* __restrict__ x,
                                       const float* __restrict__ w, float eps,
                                       float offset, int width) {
  const long row = blockIdx.x;
  const float* xr = x + row * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = xr[c];
    ss += v * v;
  }
  __shared__ float lds[16];
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    out[row * width + c] = ScalarOps<T>::from_f32(xr[c] * inv * (offset + w[c]));
}

// x += mult * (a + b); cast = T(x) when asked for
template <typename T>
__global__ void stream_add_kernel(float* __restrict__ x, const T* __restrict__ a,
                                  const T* __restrict__ b, float mult,
                                  T* __restrict__ cast, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    float s = ScalarOps<T>::to_f32(a[i]);
    if (b != nullptr) s += ScalarOps<T>::to_f32(b[i]);
    const float v = x[i] + mult * s;
    x[i] = v;
    if (cast != nullptr) cast[i] = ScalarOps<T>::from_f32(v);
  }
}

// x += mult * y / sqrt(mean(y^2) + eps) * w
template <typename T>
__global__ void stream_add_rms_norm_kernel(float* __restrict__ x,
                                           const T* __restrict__ y,
                                           const float* __restrict__ w,
                                           float eps, float mult, int width) {
  const long row = blockIdx.x;
  const T* yr = y + row * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = ScalarOps<T>::to_f32(yr[c]);
    ss += v * v;
  }
  __shared__ float lds[16];
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    x[row * width + c] += mult * (ScalarOps<T>::to_f32(yr[c]) * inv * w[c]);
}

template <typename T>
__global__ void softcap_kernel(float* __restrict__ out, const T* __restrict__ in,
                               float cap, long n) {
  const float inv = 1.0f / cap;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x)
    out[i] = cap * tanhf(ScalarOps<T>::to_f32(in[i]) * inv);
}

// Half-split rotation of dims [offset, offset + 2*half) of every head of
// x [T, H, D] (strided), in place.  Angle = float(position) * inv_freq[i].
template <typename T>
__global__ void rope_partial_kernel(T* __restrict__ x, long st, long sh,
                                    const long* __restrict__ positions,
                                    const float* __restrict__ inv_freq,
                                    int heads, int offset, int half, long n) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n;
       i += (long)gridDim.x * blockDim.x) {
    const int k = (int)(i % half);
    const long th = i / half;
    const int h = (int)(th % heads);
    const long t = th / heads;
    const float ang = (float)positions[t] * inv_freq[k];
    float s, c;
    sincosf(ang, &s, &c);
    T* p = x + t * st + h * sh + offset;
    const float u = ScalarOps<T>::to_f32(p[k]);
    const float v = ScalarOps<T>::to_f32(p[k + half]);
    p[k] = ScalarOps<T>::from_f32(u * c - v * s);
    p[k + half] = ScalarOps<T>::from_f32(v * c + u * s);
  }
}

// One workgroup per token: RMS-norm the first `rank` values of the row with a
// plain weight, rotate the first 2*half of the remaining `rot` values, store
// the row at its slot of the paged cache (slot < 0: padding row, skipped).
template <typename T>
__global__ void latent_kv_write_kernel(const T* __restrict__ dkv,
                                       const float* __restrict__ norm_w,
                                       float eps,
                                       const long* __restrict__ positions,
                                       const float* __restrict__ inv_freq,
                                       int half, T* __restrict__ cache,
                                       const long* __restrict__ slot_mapping,
                                       int rank, int rot) {
  const long t = blockIdx.x;
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  const int d = rank + rot;
  const T* in = dkv + t * d;
  T* out = cache + slot * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += blockDim.x) {
    const float v = ScalarOps<T>::to_f32(in[c]);
    ss += v * v;
  }
  __shared__ float lds[16];
  ss = block_reduce_sum(ss, lds);
  const float inv = 1.0f / sqrtf(ss / rank + eps);
  for (int c = threadIdx.x; c < rank; c += blockDim.x)
    out[c] = ScalarOps<T>::from_f32(ScalarOps<T>::to_f32(in[c]) * inv * norm_w[c]);
  const float pos = (float)positions[t];
  for (int k = threadIdx.x; k < half; k += blockDim.x) {
    float s, c;
    sincosf(pos * inv_freq[k], &s, &c);
    const float u = ScalarOps<T>::to_f32(in[rank + k]);
    const float v = ScalarOps<T>::to_f32(in[rank + k + half]);
    out[rank + k] = ScalarOps<T>::from_f32(u * c - v * s);
    out[rank + k + half] = ScalarOps<T>::from_f32(v * c + u * s);
  }
  for (int k = 2 * half + threadIdx.x; k < rot; k += blockDim.x)
    out[rank + k] = in[rank + k];
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------

static inline int grid_for(long n, int block) {
  long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

template <typename T>
void launch_gelu_tanh(T* out, const T* x, const T* mul, long mul_stride,
                      int cols, long n, hipStream_t s) {
  gelu_tanh_kernel<T><<<grid_for(n, 256), 256, 0, s>>>(out, x, mul, mul_stride, cols, n);
}
template <typename T>
void launch_embedding_scaled(float* out, const long* ids, const T* table,
                             float scale, int rows, int width, hipStream_t s) {
  embedding_scaled_kernel<T><<<rows, 256, 0, s>>>(out, ids, table, scale, width);
}
template <typename T>
void launch_rms_norm_stream(T* out, const float* x, const float* w, float eps,
                            float offset, int rows, int width, hipStream_t s) {
  rms_norm_stream_kernel<T><<<rows, 256, 0, s>>>(out, x, w, eps, offset, width);
}
template <typename T>
void launch_stream_add(float* x, const T* a, const T* b, float mult, T* cast,
                       long n, hipStream_t s) {
  stream_add_kernel<T><<<grid_for(n, 256), 256, 0, s>>>(x, a, b, mult, cast, n);
}
template <typename T>
void launch_stream_add_rms_norm(float* x, const T* y, const float* w, float eps,
                                float mult, int rows, int width, hipStream_t s) {
  stream_add_rms_norm_kernel<T><<<rows, 256, 0, s>>>(x, y, w, eps, mult, width);
}
template <typename T>
void launch_softcap(float* out, const T* in, float cap, long n, hipStream_t s) {
  softcap_kernel<T><<<grid_for(n, 256), 256, 0, s>>>(out, in, cap, n);
}
template <typename T>
void launch_rope_partial(T* x, long st, long sh, const long* positions,
                         const float* inv_freq, int rows, int heads, int offset,
                         int half, hipStream_t s) {
  const long n = (long)rows * heads * half;
  rope_partial_kernel<T><<<grid_for(n, 256), 256, 0, s>>>(
      x, st, sh, positions, inv_freq, heads, offset, half, n);
}
template <typename T>
void launch_latent_kv_write(const T* dkv, const float* norm_w, float eps,
                            const long* positions, const float* inv_freq,
                            int half, T* cache, const long* slot_mapping,
                            int rows, int rank, int rot, hipStream_t s) {
  latent_kv_write_kernel<T><<<rows, 128, 0, s>>>(
      dkv, norm_w, eps, positions, inv_freq, half, cache, slot_mapping, rank, rot);
}

#define INSTANTIATE(T)                                                          \
  template void launch_gelu_tanh<T>(T*, const T*, const T*, long, int, long,    \
                                    hipStream_t);                               \
  template void launch_embedding_scaled<T>(float*, const long*, const T*,       \
                                           float, int, int, hipStream_t);       \
  template void launch_rms_norm_stream<T>(T*, const float*, const float*,       \
                                          float, float, int, int, hipStream_t); \
  template void launch_stream_add<T>(float*, const T*, const T*, float, T*,     \
                                     long, hipStream_t);                        \
  template void launch_stream_add_rms_norm<T>(float*, const T*, const float*,   \
                                              float, float, int, int,           \
                                              hipStream_t);                     \
  template void launch_softcap<T>(float*, const T*, float, long, hipStream_t);  \
  template void launch_rope_partial<T>(T*, long, long, const long*,             \
                                       const float*, int, int, int, int,        \
                                       hipStream_t);                            \
  template void launch_latent_kv_write<T>(const T*, const float*, float,        \
                                          const long*, const float*, int, T*,   \
                                          const long*, int, int, int,           \
                                          hipStream_t);
INSTANTIATE(float)
INSTANTIATE(__hip_bfloat16)
