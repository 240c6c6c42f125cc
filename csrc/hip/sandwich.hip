// Sublayers between two layer norms on an fp32 residual stream, the per-channel causal convolution on a mixer's
// input, and the token + hashed-bigram embedding. One workgroup per token; a token's row is staged in LDS once
// and every statistic is an fp32 sum over it (mean first, then the mean of the squared deviations).
//
//   layer_norm32      h = (x - mean) / sqrt(var + eps) * w + b                          -> fp32 and / or storage type
//   gated_norm_add    x <- x + s * LN(y * sigmoid(r); w, b)   [+ the next sublayer's norm of the new x]
//   canon_conv        out_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j); history before a row's first token comes
//                     from the row's state slot (zeros before position 0); the slot then takes the row's last inputs
//   embed_bigram_norm x = LN(E[tok] + B[(prev * a + tok * b) mod n])   (row n of B at position 0)
//
// T is the storage type (bf16 / fp32) of weights and of the sublayers' outputs; the stream x is fp32.
// Rows of the packed batch: row b owns tokens cu_q[b] .. cu_q[b+1], its first token has position first_pos[b], its
// state lives in slot state_slots[b] (negative: a padding row that touches no state).
#include "common.hpp"

namespace {

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

// Four consecutive elements at index i (a multiple of 4; the pointers are 16-byte aligned and rows are multiples of 4).
template <typename T> DEVINL f32x4 ld4(const T* p, size_t i);
template <> DEVINL f32x4 ld4<bf16_t>(const bf16_t* p, size_t i) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p + i);
  return (f32x4){bf2f(v[0]), bf2f(v[1]), bf2f(v[2]), bf2f(v[3])};
}
template <> DEVINL f32x4 ld4<float>(const float* p, size_t i) { return *reinterpret_cast<const f32x4*>(p + i); }
template <typename T> DEVINL void st4(T* p, size_t i, f32x4 v);
template <> DEVINL void st4<bf16_t>(bf16_t* p, size_t i, f32x4 v) {
  *reinterpret_cast<bf16x4*>(p + i) = (bf16x4){f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}
template <> DEVINL void st4<float>(float* p, size_t i, f32x4 v) { *reinterpret_cast<f32x4*>(p + i) = v; }

// Sum over the threads of a workgroup (a multiple of 64, at most 1024); every thread gets the result. `red` holds 16
// floats. Every thread adds the waves' sums in the same order, so all of them see the same bits.
DEVINL float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) s += red[w];
  return s;
}

// (mean, 1 / sqrt(var + eps)) of the W floats in `row` (LDS); every thread gets both.
DEVINL void row_stats(const float* row, int W, float eps, float* red, float& mean, float& rstd) {
  float s = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) s += row[i];
  mean = block_sum(s, red) / (float)W;
  float v = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float d = row[i] - mean;
    v += d * d;
  }
  rstd = 1.f / sqrtf(block_sum(v, red) / (float)W + eps);
}

// Row of the packed batch that owns token t: cu_q is ascending, cu_q[0] = 0, cu_q[B] >= t + 1 for live tokens.
DEVINL int row_of(const int* __restrict__ cu_q, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_q[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

template <typename T, bool V4>
__global__ void __launch_bounds__(1024) layer_norm32_kernel(const float* __restrict__ x, const T* __restrict__ w,
                                                            const T* __restrict__ b, float* __restrict__ o32,
                                                            T* __restrict__ oc, int W, float eps) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  float* red = row + W;
  const size_t base = (size_t)blockIdx.x * W;
  if (V4) {
    for (int i = 4 * threadIdx.x; i < W; i += 4 * blockDim.x) *reinterpret_cast<f32x4*>(row + i) = ld4<float>(x, base + i);
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) row[i] = x[base + i];
  }
  __syncthreads();
  float mean, rstd;
  row_stats(row, W, eps, red, mean, rstd);
  if (V4) {
    for (int i = 4 * threadIdx.x; i < W; i += 4 * blockDim.x) {
      const f32x4 h = (*reinterpret_cast<const f32x4*>(row + i) - mean) * rstd * ld4<T>(w, i) + ld4<T>(b, i);
      if (o32) st4<float>(o32, base + i, h);
      if (oc) st4<T>(oc, base + i, h);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float h = (row[i] - mean) * rstd * ldf<T>(w, i) + ldf<T>(b, i);
      if (o32) o32[base + i] = h;
      if (oc) stf<T>(oc, base + i, h);
    }
  }
}

// V4: rows that are multiples of 4 wide move as 16-byte (fp32) / 8-byte (bf16) vectors.
template <typename T, bool V4>
__global__ void __launch_bounds__(1024) gated_norm_add_kernel(
    float* __restrict__ x, const T* __restrict__ y, const T* __restrict__ gate, const T* __restrict__ w,
    const T* __restrict__ b, const T* __restrict__ scale, const T* __restrict__ nw, const T* __restrict__ nb,
    float* __restrict__ h32, T* __restrict__ hc, int W, float eps) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  float* red = row + W;
  const size_t base = (size_t)blockIdx.x * W;
  if (V4) {
    for (int i = 4 * threadIdx.x; i < W; i += 4 * blockDim.x) {
      f32x4 z = ld4<T>(y, base + i);
      if (gate) {
        const f32x4 g = ld4<T>(gate, base + i);
#pragma unroll
        for (int k = 0; k < 4; ++k) z[k] /= 1.f + expf(-g[k]);
      }
      *reinterpret_cast<f32x4*>(row + i) = z;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float z = ldf<T>(y, base + i);
      if (gate) z /= 1.f + expf(-ldf<T>(gate, base + i));
      row[i] = z;
    }
  }
  __syncthreads();
  float mean, rstd;
  row_stats(row, W, eps, red, mean, rstd);
  if (V4) {
    for (int i = 4 * threadIdx.x; i < W; i += 4 * blockDim.x) {
      f32x4 r = (*reinterpret_cast<const f32x4*>(row + i) - mean) * rstd * ld4<T>(w, i) + ld4<T>(b, i);
      if (scale) r *= ld4<T>(scale, i);
      const f32x4 nx = ld4<float>(x, base + i) + r;
      st4<float>(x, base + i, nx);
      *reinterpret_cast<f32x4*>(row + i) = nx;  // the elements this thread owns in every pass
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float r = (row[i] - mean) * rstd * ldf<T>(w, i) + ldf<T>(b, i);
      if (scale) r *= ldf<T>(scale, i);
      const float nx = x[base + i] + r;
      x[base + i] = nx;
      row[i] = nx;  // the element this thread owns in every pass
    }
  }
  if (!nw) return;
  __syncthreads();
  row_stats(row, W, eps, red, mean, rstd);
  if (V4) {
    for (int i = 4 * threadIdx.x; i < W; i += 4 * blockDim.x) {
      const f32x4 h = (*reinterpret_cast<const f32x4*>(row + i) - mean) * rstd * ld4<T>(nw, i) + ld4<T>(nb, i);
      if (h32) st4<float>(h32, base + i, h);
      if (hc) st4<T>(hc, base + i, h);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float h = (row[i] - mean) * rstd * ldf<T>(nw, i) + ldf<T>(nb, i);
      if (h32) h32[base + i] = h;
      if (hc) stf<T>(hc, base + i, h);
    }
  }
}

// One workgroup per token. The workgroup of a row's FIRST token also serves the row's next taps - 2 tokens (all those
// whose history reaches into the state slot) and then rewrites the slot, so nobody else reads or writes that slot.
template <typename T>
__global__ void __launch_bounds__(256) canon_conv_kernel(const float* __restrict__ h, const T* __restrict__ w,
                                                         float* __restrict__ state, const int* __restrict__ cu_q,
                                                         const int* __restrict__ first_pos,
                                                         const int* __restrict__ state_slots, T* __restrict__ out,
                                                         int B, int W, int taps) {
  const int t = blockIdx.x, K = taps - 1, c = blockIdx.y * 256 + threadIdx.x;  // one channel per thread
  const int b = row_of(cu_q, B, t);
  const int q0 = cu_q[b], n = cu_q[b + 1] - q0, off = t - q0;
  if (off >= n) return;  // a token no row owns
  const int slot = state_slots[b];
  if (slot < 0) {  // padding row: its values go nowhere, they only have to be finite
    if (c < W) stf<T>(out, (size_t)t * W + c, h[(size_t)t * W + c]);
    return;
  }
  if (off >= K) {  // the whole history is inside the row
    if (c < W) {
      float a = h[(size_t)t * W + c];
      for (int j = 0; j < taps; ++j) a += ldf<T>(w, (size_t)c * taps + j) * h[(size_t)(t - K + j) * W + c];
      stf<T>(out, (size_t)t * W + c, a);
    }
    return;
  }
  if (off > 0) return;  // served by the workgroup of the row's first token
  const int p0 = first_pos[b];
  float* sl = state + (size_t)slot * K * W;
  // input at index p relative to the row's first token (p < 0: the state slot, or zero before the sequence's start)
  auto val = [&](int p, int c) -> float {
    if (p >= 0) return h[(size_t)(q0 + p) * W + c];
    return p0 + p >= 0 ? sl[(size_t)(K + p) * W + c] : 0.f;
  };
  const int m = min(K, n);
  if (c < W) {
    for (int i = 0; i < m; ++i) {
      float a = val(i, c);
      for (int j = 0; j < taps; ++j) a += ldf<T>(w, (size_t)c * taps + j) * val(i - K + j, c);
      stf<T>(out, (size_t)(q0 + i) * W + c, a);
    }
    // the slot's entry k becomes the input K - k tokens before the NEXT token; reads run ahead of the writes
    for (int k = 0; k < K; ++k) sl[(size_t)k * W + c] = val(n - K + k, c);
  }
}

template <typename T>
__global__ void __launch_bounds__(1024) embed_bigram_norm_kernel(
    const int64_t* __restrict__ tokens, const T* __restrict__ embed, const T* __restrict__ bigram, int buckets,
    int64_t mul_prev, int64_t mul_cur, const T* __restrict__ w, const T* __restrict__ bias, float eps,
    const int* __restrict__ cu_q, const int* __restrict__ first_pos, const int* __restrict__ state_slots,
    int* __restrict__ prev_state, float* __restrict__ out, int B, int W, int vocab) {
  extern __shared__ float row[];
  float* red = row + W;
  __shared__ int64_t big_row;
  const int t = blockIdx.x;
  int64_t tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  if (threadIdx.x == 0) {
    int64_t r = -1;
    if (bigram) {
      const int b = row_of(cu_q, B, t);
      const int q0 = cu_q[b], n = cu_q[b + 1] - q0, off = t - q0, slot = state_slots[b];
      if (off < n && slot >= 0) {
        if (first_pos[b] + off == 0) {
          r = buckets;
        } else {
          const int64_t prev = off > 0 ? tokens[t - 1] : (int64_t)prev_state[slot];
          r = (prev * mul_prev + tok * mul_cur) % (int64_t)buckets;
          if (r < 0) r += buckets;
        }
        // the row's first token owns the slot: it has read the token before, now it leaves the row's last one
        if (off == 0) prev_state[slot] = (int)tokens[q0 + n - 1];
      }
    }
    big_row = r;
  }
  __syncthreads();
  const int64_t r = big_row;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = ldf<T>(embed, (size_t)tok * W + i);
    if (r >= 0) v += ldf<T>(bigram, (size_t)r * W + i);
    row[i] = v;
  }
  __syncthreads();
  float mean, rstd;
  row_stats(row, W, eps, red, mean, rstd);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    out[(size_t)t * W + i] = (row[i] - mean) * rstd * ldf<T>(w, i) + ldf<T>(bias, i);
}

}  // namespace

// Threads of a one-token workgroup: a few elements per thread, so that a launch of few tokens (a decode step) is not a
// chain of dependent loads.
static int row_threads(int W) { return W > 2048 ? 1024 : (W > 512 ? 512 : 256); }

static int row_lds(int W, size_t* bytes) {
  *bytes = (size_t)(W + 16) * sizeof(float);
  return *bytes <= 64 * 1024 ? 0 : -2;  // rows up to 16368 channels
}

// Threads of a one-token workgroup in the vector variants: four elements a thread and pass where the row allows.
static int row_threads4(int W) {
  const int t = ((W / 4 + 63) / 64) * 64;
  return t > 1024 ? 1024 : (t < 64 ? 64 : t);
}
static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

extern "C" int areal_layer_norm32(const float* x, const void* w, const void* b, float* o32, void* oc, int T, int W,
                                  float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  size_t lds;
  if (W <= 0 || row_lds(W, &lds)) return -2;
  const bool v4 = W % 4 == 0 && aligned16(x) && aligned16(w) && aligned16(b) && aligned16(o32) && aligned16(oc);
#define LN_LAUNCH(TT, V4, NTHR)                                                                               \
  hipLaunchKernelGGL((layer_norm32_kernel<TT, V4>), dim3(T), dim3(NTHR), lds, st, x, (const TT*)w, (const TT*)b, \
                     o32, (TT*)(dt == 0 ? oc : nullptr), W, eps)
  if (dt == 0) {
    if (v4) LN_LAUNCH(bf16_t, true, row_threads4(W));
    else LN_LAUNCH(bf16_t, false, row_threads(W));
  } else {
    if (v4) LN_LAUNCH(float, true, row_threads4(W));
    else LN_LAUNCH(float, false, row_threads(W));
  }
#undef LN_LAUNCH
  return (int)hipGetLastError();
}

extern "C" int areal_gated_norm_add(float* x, const void* y, const void* gate, const void* w, const void* b,
                                    const void* scale, const void* nw, const void* nb, float* h32, void* hc, int T,
                                    int W, float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  size_t lds;
  if (W <= 0 || row_lds(W, &lds)) return -2;
  const bool v4 = W % 4 == 0 && aligned16(x) && aligned16(y) && aligned16(gate) && aligned16(w) && aligned16(b) &&
                  aligned16(scale) && aligned16(nw) && aligned16(nb) && aligned16(h32) && aligned16(hc);
#define GN_LAUNCH(TT, V4, NTHR)                                                                                  \
  hipLaunchKernelGGL((gated_norm_add_kernel<TT, V4>), dim3(T), dim3(NTHR), lds, st, x, (const TT*)y,             \
                     (const TT*)gate, (const TT*)w, (const TT*)b, (const TT*)scale, (const TT*)nw, (const TT*)nb, \
                     h32, (TT*)(dt == 0 ? hc : nullptr), W, eps)
  if (dt == 0) {
    if (v4) GN_LAUNCH(bf16_t, true, row_threads4(W));
    else GN_LAUNCH(bf16_t, false, row_threads(W));
  } else {
    if (v4) GN_LAUNCH(float, true, row_threads4(W));
    else GN_LAUNCH(float, false, row_threads(W));
  }
#undef GN_LAUNCH
  return (int)hipGetLastError();
}

extern "C" int areal_canon_conv(const float* h, const void* w, float* state, const int* cu_q, const int* first_pos,
                                const int* state_slots, void* out, int B, int T, int W, int taps, int dt,
                                hipStream_t st) {
  if (T == 0 || B == 0) return 0;
  if (taps < 1 || (taps > 1 && !state) || (W + 255) / 256 > 65535) return -1;
  if (dt == 0)
    hipLaunchKernelGGL(canon_conv_kernel<bf16_t>, dim3(T, (W + 255) / 256), dim3(256), 0, st, h, (const bf16_t*)w, state, cu_q,
                       first_pos, state_slots, (bf16_t*)out, B, W, taps);
  else
    hipLaunchKernelGGL(canon_conv_kernel<float>, dim3(T, (W + 255) / 256), dim3(256), 0, st, h, (const float*)w, state, cu_q,
                       first_pos, state_slots, (float*)out, B, W, taps);
  return (int)hipGetLastError();
}

extern "C" int areal_embed_bigram_norm(const int64_t* tokens, const void* embed, const void* bigram, int buckets,
                                       int64_t mul_prev, int64_t mul_cur, const void* w, const void* bias, float eps,
                                       const int* cu_q, const int* first_pos, const int* state_slots, int* prev_state,
                                       float* out, int B, int T, int W, int vocab, int dt, hipStream_t st) {
  if (T == 0 || B == 0) return 0;
  size_t lds;
  if (W <= 0 || row_lds(W, &lds)) return -2;
  if (bigram && (buckets < 1 || !prev_state)) return -1;
  if (dt == 0)
    hipLaunchKernelGGL(embed_bigram_norm_kernel<bf16_t>, dim3(T), dim3(row_threads(W)), lds, st, tokens, (const bf16_t*)embed,
                       (const bf16_t*)bigram, buckets, mul_prev, mul_cur, (const bf16_t*)w, (const bf16_t*)bias, eps,
                       cu_q, first_pos, state_slots, prev_state, out, B, W, vocab);
  else
    hipLaunchKernelGGL(embed_bigram_norm_kernel<float>, dim3(T), dim3(row_threads(W)), lds, st, tokens, (const float*)embed,
                       (const float*)bigram, buckets, mul_prev, mul_cur, (const float*)w, (const float*)bias, eps,
                       cu_q, first_pos, state_slots, prev_state, out, B, W, vocab);
  return (int)hipGetLastError();
}
