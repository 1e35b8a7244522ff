// Short depthwise causal convolution over time with per-sequence state.
//
//   out_t = act([h_t +] sum_j w[:, j] * h_(t - taps + 1 + j) [+ bias])
//
// act is the identity or silu; the input rows may be a column slice of a wider
// matrix (row stride in_st), output and state rows are dense.
//
// A step brings, for each sequence, rows [loc[s], loc[s+1]) of new inputs that
// continue the sequence at position start = seq_len - n.  Inputs older than the
// step's rows come from state[slot] (the last taps-1 inputs, row j holding
// position start - (taps-1) + j); positions before 0 are zero and are never
// read from the state, so a reused slot needs no clearing.  A second kernel on
// the same stream advances the state past the new rows: row j of the new state
// is position end - (taps-1) + j, taken from the step's rows or, when the step
// is shorter than taps-1, from old state row j + n — each thread walks j
// upwards, so it reads row j + n before that row is overwritten.
//
// One thread per (row, 4 channels) — or one channel when the width is not a
// multiple of 4: consecutive threads take consecutive channels,
// every load and store is coalesced; accumulation is f32.

#include "common.h"

template <typename T, int CH>
DEVINLINE void load_ch(const T* p, float* v) {
  if (CH == 4) {
    if (sizeof(T) == 4) {
      const float4 t = *reinterpret_cast<const float4*>(p);
      v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else {
      const uint2 t = *reinterpret_cast<const uint2*>(p);
      v[0] = __uint_as_float(t.x << 16);
      v[1] = __uint_as_float(t.x & 0xffff0000u);
      v[2] = __uint_as_float(t.y << 16);
      v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
  } else {
    v[0] = ScalarOps<T>::to_f32(p[0]);
  }
}

template <typename T, int CH>
DEVINLINE void store_ch(T* p, const float* v) {
#pragma unroll
  for (int k = 0; k < CH; ++k) p[k] = ScalarOps<T>::from_f32(v[k]);
}

DEVINLINE int find_seq(const int* __restrict__ loc, int nseq, int row) {
  int lo = 0, hi = nseq;  // largest s with loc[s] <= row
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (loc[mid] <= row) lo = mid; else hi = mid;
  }
  return lo;
}

// CH channels per thread: 4 (8/16-byte accesses) when width % 4 == 0, else 1.
// TAPS > 0: tap count known at compile time — the thread's CH x TAPS weights
// are one contiguous run fetched with 16-byte loads into registers; TAPS == 0
// reads them one by one for any tap count.
template <typename T, int CH, int TAPS>
__global__ void causal_conv_kernel(T* __restrict__ out, const T* __restrict__ h,
                                   const float* __restrict__ w,   // [W, taps]
                                   const T* __restrict__ state,   // [slots, taps-1, W]
                                   const int* __restrict__ loc,
                                   const int* __restrict__ seq_lens,
                                   const int* __restrict__ slots, int nseq,
                                   int width, int taps, int add_input,
                                   long in_st, const float* __restrict__ bias,
                                   int act) {
  const int row = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * CH;
  if (c >= width) return;
  const int s = find_seq(loc, nseq, row);
  const int slot = slots[s];
  const long o = (long)row * width + c;
  float acc[CH];
  if (slot < 0) {  // padding row of a captured bucket
#pragma unroll
    for (int k = 0; k < CH; ++k) acc[k] = 0.f;
    store_ch<T, CH>(out + o, acc);
    return;
  }
  const int n = loc[s + 1] - loc[s];
  const int start = seq_lens[s] - n;
  const int p = start + (row - loc[s]);
  const T* st = state + (long)slot * (taps - 1) * width;
  float wreg[CH * (TAPS > 0 ? TAPS : 1)];
  if (TAPS > 0 && CH == 4) {
#pragma unroll
    for (int i = 0; i < TAPS; ++i) {
      const float4 t = reinterpret_cast<const float4*>(w + (long)c * TAPS)[i];
      wreg[4 * i] = t.x; wreg[4 * i + 1] = t.y; wreg[4 * i + 2] = t.z; wreg[4 * i + 3] = t.w;
    }
  }
  if (add_input) {
    load_ch<T, CH>(h + (long)row * in_st + c, acc);
  } else {
#pragma unroll
    for (int k = 0; k < CH; ++k) acc[k] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < (TAPS > 0 ? TAPS : taps); ++j) {
    const int pj = p - (taps - 1) + j;
    if (pj < 0) continue;
    float v[CH];
    if (pj >= start)
      load_ch<T, CH>(h + (long)(loc[s] + pj - start) * in_st + c, v);
    else
      load_ch<T, CH>(st + (long)(pj - (start - (taps - 1))) * width + c, v);
#pragma unroll
    for (int k = 0; k < CH; ++k) {
      const float wk = (TAPS > 0 && CH == 4) ? wreg[k * TAPS + j] : w[(c + k) * taps + j];
      acc[k] += wk * v[k];
    }
  }
  if (bias != nullptr) {
#pragma unroll
    for (int k = 0; k < CH; ++k) acc[k] += bias[c + k];
  }
  if (act == 1) {
#pragma unroll
    for (int k = 0; k < CH; ++k) acc[k] = acc[k] / (1.0f + expf(-acc[k]));
  }
  store_ch<T, CH>(out + o, acc);
}

template <typename T>
__global__ void conv_state_update_kernel(T* __restrict__ state,
                                         const T* __restrict__ h,
                                         const int* __restrict__ loc,
                                         const int* __restrict__ seq_lens,
                                         const int* __restrict__ slots,
                                         int width, int taps, long in_st) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int slot = slots[s];
  if (slot < 0) return;
  const int n = loc[s + 1] - loc[s];
  if (n <= 0) return;
  const int end = seq_lens[s];
  const int start = end - n;
  T* st = state + (long)slot * (taps - 1) * width;
  for (int j = 0; j < taps - 1; ++j) {
    const int pj = end - (taps - 1) + j;
    T v = ScalarOps<T>::from_f32(0.f);
    if (pj >= start)
      v = h[(long)(loc[s] + pj - start) * in_st + c];
    else if (pj >= 0)
      v = st[(long)(j + n) * width + c];
    st[(long)j * width + c] = v;
  }
}

template <typename T>
void launch_causal_conv_state(T* out, const T* h, const float* w, T* state,
                              const int* loc, const int* seq_lens,
                              const int* slots, int rows, int nseq, int width,
                              int taps, int add_input, long in_st,
                              const float* bias, int act, hipStream_t stream) {
  const int block = 256;
  const bool vec = width % 4 == 0 && in_st % 4 == 0 &&
                   (bias == nullptr || reinterpret_cast<uintptr_t>(bias) % 16 == 0) &&
                   reinterpret_cast<uintptr_t>(h) % (4 * sizeof(T)) == 0 &&
                   reinterpret_cast<uintptr_t>(state) % (4 * sizeof(T)) == 0 &&
                   reinterpret_cast<uintptr_t>(w) % 16 == 0;
  if (vec) {
    dim3 g1(rows, (width / 4 + block - 1) / block);
#define CONV_LAUNCH(TP)                                                        \
    causal_conv_kernel<T, 4, TP><<<g1, block, 0, stream>>>(                    \
        out, h, w, state, loc, seq_lens, slots, nseq, width, taps, add_input, \
        in_st, bias, act)
    switch (taps) {
      case 2: CONV_LAUNCH(2); break;
      case 3: CONV_LAUNCH(3); break;
      case 4: CONV_LAUNCH(4); break;
      default: CONV_LAUNCH(0); break;
    }
#undef CONV_LAUNCH
  } else {
    dim3 g1(rows, (width + block - 1) / block);
    causal_conv_kernel<T, 1, 0><<<g1, block, 0, stream>>>(
        out, h, w, state, loc, seq_lens, slots, nseq, width, taps, add_input,
        in_st, bias, act);
  }
  if (taps > 1) {
    dim3 g2(nseq, (width + block - 1) / block);
    conv_state_update_kernel<T><<<g2, block, 0, stream>>>(
        state, h, loc, seq_lens, slots, width, taps, in_st);
  }
}

template void launch_causal_conv_state<float>(float*, const float*, const float*,
                                              float*, const int*, const int*,
                                              const int*, int, int, int, int,
                                              int, long, const float*, int,
                                              hipStream_t);
template void launch_causal_conv_state<__hip_bfloat16>(
    __hip_bfloat16*, const __hip_bfloat16*, const float*, __hip_bfloat16*,
    const int*, const int*, const int*, int, int, int, int, int, long,
    const float*, int, hipStream_t);
