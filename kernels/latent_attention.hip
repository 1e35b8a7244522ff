// Windowed multi-query attention with softmax sinks over a paged latent cache.
//
// The cache holds one row per token, [rank + rot]: a latent c and a rotated
// key part.  Every head scores the same row, (q_lat . c + q_rot . k_rot) *
// scale, and sums the same c; the softmax denominator of head h additionally
// holds exp(sink_h) (no key, no value).  A query at position i sees keys
// j with 0 <= i - j < window (window 0: every j <= i).
//
// This file is the general kernel: any rank / rot / block size, f32 or bf16
// storage, f32 scores, softmax and accumulation.  One workgroup per (query
// row, head).  Per tile of 256 keys:
//   phase 1  thread j scores key j (q broadcast from LDS, the key row read
//            with 16-byte loads), block max / sum give the online-softmax step
//   phase 2  threads are regrouped as (group g, dim k): group g accumulates
//            p_j * c_j[k] over the keys j = g mod G of the tile — loads of
//            c_j[k] are coalesced over k
// The groups are summed through LDS at the end, the sink joins the
// denominator, and the row is written with the caller's strides.
// Decode (one query per sequence) and prompt portions (rows located through
// query_start_loc) share the kernel; what differs is how a row finds its
// sequence and its context length.

#include "common.h"

#define LA_THREADS 256
#define LA_MAX_DPT 4   // output dims per thread: rank <= 256 * 4

DEVINLINE float block_reduce_max(float x, float* lds_scratch) {
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int nwaves = blockDim.x / WAVE_SIZE;
  x = wave_reduce_max(x);
  __syncthreads();
  if (lane == 0) lds_scratch[wave] = x;
  __syncthreads();
  float m = -INFINITY;
  for (int i = 0; i < nwaves; ++i) m = fmaxf(m, lds_scratch[i]);
  __syncthreads();
  return m;
}

DEVINLINE float block_reduce_sum2(float x, float* lds_scratch) {
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int nwaves = blockDim.x / WAVE_SIZE;
  x = wave_reduce_sum(x);
  __syncthreads();
  if (lane == 0) lds_scratch[wave] = x;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nwaves; ++i) s += lds_scratch[i];
  __syncthreads();
  return s;
}

template <typename T>
__global__ __launch_bounds__(LA_THREADS) void latent_attn_row_kernel(
    T* __restrict__ out, long o_st, long o_sh,
    const T* __restrict__ q_lat, long ql_st, long ql_sh,
    const T* __restrict__ q_rot, long qr_st, long qr_sh,
    const T* __restrict__ cache, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    int nseq, const float* __restrict__ sinks, float scale, int window,
    int rank, int rot, int block_size, int rp /* pow2 >= min(rank,256) */) {
  extern __shared__ float smem[];
  const int d = rank + rot;
  float* q_s = smem;                  // [d]
  float* p_s = q_s + ((d + 1) & ~1);  // [256]; keeps off_s 8-byte aligned
  long* off_s = reinterpret_cast<long*>(p_s + LA_THREADS);   // [256]
  float* red = reinterpret_cast<float*>(off_s + LA_THREADS); // [16]
  float* acc_s = red + 16;            // [256] cross-group sums

  const int row = blockIdx.x;
  const int h = blockIdx.y;
  const int tid = threadIdx.x;

  int seq, ctx;
  if (qsl != nullptr) {
    int lo = 0, hi = nseq;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (qsl[mid] <= row) lo = mid; else hi = mid;
    }
    seq = lo;
    const int n = qsl[seq + 1] - qsl[seq];
    ctx = seq_lens[seq] - n + (row - qsl[seq]) + 1;
  } else {
    seq = row;
    ctx = seq_lens[row];
  }
  T* orow = out + row * o_st + h * o_sh;
  if (ctx <= 0) {
    for (int k = tid; k < rank; k += LA_THREADS) orow[k] = ScalarOps<T>::from_f32(0.f);
    return;
  }
  const int first = (window > 0 && ctx > window) ? ctx - window : 0;

  const T* ql = q_lat + row * ql_st + h * ql_sh;
  const T* qr = q_rot + row * qr_st + h * qr_sh;
  for (int k = tid; k < rank; k += LA_THREADS) q_s[k] = ScalarOps<T>::to_f32(ql[k]) * scale;
  for (int k = tid; k < rot; k += LA_THREADS) q_s[rank + k] = ScalarOps<T>::to_f32(qr[k]) * scale;
  __syncthreads();

  constexpr int V = Vec16<T>::kElems;
  const bool vec_ok = (d % V) == 0;
  const int* bt = block_tables + (long)seq * bt_stride;

  const int groups = LA_THREADS / rp;       // >= 1
  const int g = tid / rp;
  const int k0 = tid - g * rp;
  float acc[LA_MAX_DPT];
#pragma unroll
  for (int i = 0; i < LA_MAX_DPT; ++i) acc[i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  for (int base = first; base < ctx; base += LA_THREADS) {
    const int j = base + tid;
    float s = -INFINITY;
    if (j < ctx) {
      const long off = ((long)bt[j / block_size] * block_size + (j % block_size)) * d;
      off_s[tid] = off;
      const T* kr = cache + off;
      float a = 0.f;
      if (vec_ok) {
        for (int k = 0; k < d; k += V) {
          const Vec16<T> v = load16(kr + k);
#pragma unroll
          for (int u = 0; u < V; ++u) a += q_s[k + u] * ScalarOps<T>::to_f32(v.data[u]);
        }
      } else {
        for (int k = 0; k < d; ++k) a += q_s[k] * ScalarOps<T>::to_f32(kr[k]);
      }
      s = a;
    }
    const float m_tile = block_reduce_max(s, red);
    const float m_new = fmaxf(m_run, m_tile);
    const float alpha = (m_run == -INFINITY) ? 0.f : expf(m_run - m_new);
    const float p = (j < ctx) ? expf(s - m_new) : 0.f;
    p_s[tid] = p;
    const float l_tile = block_reduce_sum2(p, red);   // barriers also publish p_s/off_s
    l_run = l_run * alpha + l_tile;
    m_run = m_new;
    const int nk = min(LA_THREADS, ctx - base);
#pragma unroll
    for (int i = 0; i < LA_MAX_DPT; ++i) acc[i] *= alpha;
    for (int jj = g; jj < nk; jj += groups) {
      const float pj = p_s[jj];
      const T* cr = cache + off_s[jj];
#pragma unroll
      for (int i = 0; i < LA_MAX_DPT; ++i) {
        const int k = k0 + i * rp;
        if (k < rank) acc[i] += pj * ScalarOps<T>::to_f32(cr[k]);
      }
    }
    __syncthreads();   // p_s / off_s are rewritten by the next tile
  }

  float m_fin = m_run, l_fin = l_run, rescale = 1.f;
  if (sinks != nullptr) {
    const float sk = sinks[h];
    m_fin = fmaxf(m_run, sk);
    rescale = expf(m_run - m_fin);
    l_fin = l_run * rescale + expf(sk - m_fin);
  }
  const float inv = rescale / l_fin;

  if (groups > 1) {
    // rank <= rp <= 128 here: one dim per thread, sum the groups through LDS
    acc_s[tid] = acc[0];
    __syncthreads();
    if (g == 0 && k0 < rank) {
      float a = 0.f;
      for (int gg = 0; gg < groups; ++gg) a += acc_s[gg * rp + k0];
      orow[k0] = ScalarOps<T>::from_f32(a * inv);
    }
  } else {
#pragma unroll
    for (int i = 0; i < LA_MAX_DPT; ++i) {
      const int k = k0 + i * rp;
      if (k < rank) orow[k] = ScalarOps<T>::from_f32(acc[i] * inv);
    }
  }
}

template <typename T>
void launch_latent_attention(T* out, long o_st, long o_sh, const T* q_lat,
                             long ql_st, long ql_sh, const T* q_rot, long qr_st,
                             long qr_sh, const T* cache, const int* block_tables,
                             int bt_stride, const int* qsl, const int* seq_lens,
                             int nseq, const float* sinks, float scale,
                             int window, int rows, int heads, int rank, int rot,
                             int block_size, hipStream_t stream) {
  int rp = 1;
  while (rp < rank && rp < LA_THREADS) rp <<= 1;
  const int d = rank + rot;
  const size_t smem = sizeof(float) * (((d + 1) & ~1) + LA_THREADS + 16 + LA_THREADS) +
                      sizeof(long) * LA_THREADS;
  dim3 grid(rows, heads);
  latent_attn_row_kernel<T><<<grid, LA_THREADS, smem, stream>>>(
      out, o_st, o_sh, q_lat, ql_st, ql_sh, q_rot, qr_st, qr_sh, cache,
      block_tables, bt_stride, qsl, seq_lens, nseq, sinks, scale, window, rank,
      rot, block_size, rp);
}

template void launch_latent_attention<float>(
    float*, long, long, const float*, long, long, const float*, long, long,
    const float*, const int*, int, const int*, const int*, int, const float*,
    float, int, int, int, int, int, int, hipStream_t);
template void launch_latent_attention<__hip_bfloat16>(
    __hip_bfloat16*, long, long, const __hip_bfloat16*, long, long,
    const __hip_bfloat16*, long, long, const __hip_bfloat16*, const int*, int,
    const int*, const int*, int, const float*, float, int, int, int, int, int,
    int, hipStream_t);
