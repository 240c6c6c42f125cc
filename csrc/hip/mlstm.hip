// Matrix-memory recurrence (mLSTM of the xLSTM family) with a carried, stabilised fp32 state.
//
// Per head, with log gates i_t, f_t (fp32), keys / queries of size D and values of size V:
//
//   m_t = max(f_t + m_{t-1}, i_t)                      a_t = exp(f_t + m_{t-1} - m_t),  b_t = exp(i_t - m_t)
//   S_t = a_t S_{t-1} + b_t k_t v_t^T   [D, V]         n_t = a_t n_{t-1} + b_t k_t   [D]
//   y_t = S_t^T (q_t / sqrt(D)) / (max(|n_t . q_t / sqrt(D)|, exp(-m_t)) + 1e-6)
//
// State slots [slots, heads, ...] live in device memory between steps: a row whose first token has position 0
// starts from S = 0, n = 0, m = 0 whatever its slot held before; a row with a negative slot is skipped.
//
// `mlstm_gates`: i = cap tanh((W_i x + b_i) / cap), f = logsigmoid(cap tanh((W_f x + b_f) / cap)) with fp32
// accumulation of the dot products (the gates enter exponentials of running sums, so they never pass through bf16).
// `mlstm_scan`: one workgroup of four waves per (row, head, 64 value columns); every wave keeps a quarter of the
// rows of S (lane c: column c) and of n in registers; keys and queries of a few tokens at a time are staged in LDS as
// fp32. It writes the unnormalised read-out S_t^T q_t, n_t . q_t and m_t; `mlstm_out` divides, applies the per-head RMS norm,
// the weight and the sigmoid output gate.
#include "common.hpp"

namespace {

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

// w [2 * NH, W]: rows of the input gate's heads, then of the forget gate's; b [2 * NH]. A workgroup takes GT tokens
// and four gate rows (one a wave), so a weight row is read once per GT tokens; decode batches run GT = 1 for the
// sake of more workgroups.
template <typename T, int GT>
__global__ void __launch_bounds__(256) mlstm_gates_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                           const T* __restrict__ bias, float* __restrict__ ig,
                                                           float* __restrict__ fg, int Ttok, int W, int NH, float cap) {
  const int t0 = blockIdx.x * GT, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int u = blockIdx.y * 4 + wave;
  if (u >= 2 * NH) return;
  const T* wr = w + (size_t)u * W;
  float s[GT];
#pragma unroll
  for (int tt = 0; tt < GT; ++tt) s[tt] = 0.f;
  for (int i = lane; i < W; i += 64) {
    const float wv = ldf<T>(wr, i);
#pragma unroll
    for (int tt = 0; tt < GT; ++tt) s[tt] += ldf<T>(x, (size_t)min(t0 + tt, Ttok - 1) * W + i) * wv;
  }
#pragma unroll
  for (int tt = 0; tt < GT; ++tt) {
    const float tot = wave_sum(s[tt]);
    const int t = t0 + tt;
    if (lane == 0 && t < Ttok) {
      float z = tot + (bias ? ldf<T>(bias, u) : 0.f);
      if (cap > 0.f) z = cap * tanhf(z / cap);
      if (u < NH) ig[(size_t)t * NH + u] = z;
      else fg[(size_t)t * NH + (u - NH)] = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));  // log sigmoid
    }
  }
}

constexpr int TC = 8;  // tokens staged per step of the loop
constexpr int RW = 4;  // waves of a workgroup: each keeps a quarter of the state's rows

// One workgroup per (row, head, 64 value columns). Wave r keeps rows r DQ .. r DQ + DQ - 1 of S (lane c: column c) and
// of n (lane i: row i of its quarter) in registers. Per step of TC tokens every wave forms its partial read-outs,
// the partials meet in LDS and wave r finishes tokens r and r + RW.
template <typename T, int DP>
__global__ void __launch_bounds__(64 * RW) mlstm_scan_kernel(
    const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* __restrict__ ig,
    const float* __restrict__ fg, const int* __restrict__ cu_q, const int* __restrict__ first_pos,
    const int* __restrict__ state_slots, float* __restrict__ S, float* __restrict__ N, float* __restrict__ M,
    float* __restrict__ hbuf, float* __restrict__ nq, float* __restrict__ mt, int NH, int D, int V) {
  constexpr int DQ = DP / RW;
  __shared__ float kq[TC][2][DP];
  __shared__ float hpart[RW][TC][64];
  __shared__ float npart[RW][TC];
  const int b = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x, lane = tid & 63, r = tid >> 6;
  const int col = blockIdx.z * 64 + lane;
  const bool has = col < V;
  const int slot = state_slots[b];
  const int t_lo = cu_q[b], t_hi = cu_q[b + 1];
  if (slot < 0) {  // a retired row: its outputs are defined (zero), no slot is touched
    if (r == 0)
      for (int t = t_lo; t < t_hi; ++t) {
        if (has) hbuf[((size_t)t * NH + hd) * V + col] = 0.f;
        if (blockIdx.z == 0 && lane == 0) nq[(size_t)t * NH + hd] = mt[(size_t)t * NH + hd] = 0.f;
      }
    return;
  }
  if (t_hi <= t_lo) return;
  const bool fresh = first_pos[b] == 0;
  const size_t sbase = ((size_t)slot * NH + hd) * D;
  const int d0 = r * DQ;
  float s[DQ];
#pragma unroll
  for (int d = 0; d < DQ; ++d) s[d] = (!fresh && has && d0 + d < D) ? S[(sbase + d0 + d) * V + col] : 0.f;
  const int nd = d0 + lane;  // the row of n this lane keeps
  const bool nlive = lane < DQ && nd < D;
  float nn = (!fresh && nlive) ? N[sbase + nd] : 0.f;
  float m = fresh ? 0.f : M[(size_t)slot * NH + hd];
  const float qscale = 1.f / sqrtf((float)D);
  // operands of TC tokens are fetched into registers one step ahead, so the loads' latency runs under the
  // recurrence of the tokens before
  constexpr int KQN = (TC * DP + 64 * RW - 1) / (64 * RW);
  float pk[KQN], pq[KQN], pv[TC], pf[TC], pi[TC];
  auto fetch = [&](int tb) {
    const int nt = min(TC, t_hi - tb);
#pragma unroll
    for (int j = 0; j < KQN; ++j) {
      const int i = tid + j * 64 * RW, d = i % DP, tt = i / DP;
      const bool live = tt < nt && d < D;
      const T* row = proj + (size_t)(tb + min(tt, nt - 1)) * row_stride;
      pk[j] = live ? ldf<T>(row, k_off + hd * D + d) : 0.f;
      pq[j] = live ? ldf<T>(row, q_off + hd * D + d) * qscale : 0.f;
    }
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      pv[tt] = (tt < nt && has) ? ldf<T>(proj + (size_t)(tb + tt) * row_stride, v_off + hd * V + col) : 0.f;
      pf[tt] = tt < nt ? fg[(size_t)(tb + tt) * NH + hd] : 0.f;
      pi[tt] = tt < nt ? ig[(size_t)(tb + tt) * NH + hd] : 0.f;
    }
  };
  fetch(t_lo);
  for (int tb = t_lo; tb < t_hi; tb += TC) {
    const int nt = min(TC, t_hi - tb);
    __syncthreads();  // the step before is finished with kq and the partials
#pragma unroll
    for (int j = 0; j < KQN; ++j) {
      const int i = tid + j * 64 * RW;
      if (i < TC * DP) {
        kq[i / DP][0][i % DP] = pk[j];
        kq[i / DP][1][i % DP] = pq[j];
      }
    }
    float vv[TC], fgr[TC], igr[TC];
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      vv[tt] = pv[tt];
      fgr[tt] = pf[tt];
      igr[tt] = pi[tt];
    }
    if (tb + TC < t_hi) fetch(tb + TC);
    __syncthreads();
    float mloc[TC];
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      mloc[tt] = m;
      if (tt < nt) {
        const float f = fgr[tt], ii = igr[tt];
        const float m2 = fmaxf(f + m, ii);
        const float a = expf(f + m - m2), bb = expf(ii - m2);
        m = m2;
        mloc[tt] = m;
        const float bv = bb * vv[tt];
        float hacc = 0.f;
#pragma unroll
        for (int d = 0; d < DQ; ++d) {
          s[d] = a * s[d] + bv * kq[tt][0][d0 + d];
          hacc += s[d] * kq[tt][1][d0 + d];
        }
        float part = 0.f;
        if (lane < DQ) {
          nn = a * nn + bb * kq[tt][0][nd];
          part = nn * kq[tt][1][nd];
        }
        part = wave_sum(part);
        hpart[r][tt][lane] = hacc;
        if (lane == 0) npart[r][tt] = part;
      }
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < TC; ++tt) {
      if (tt < nt && (tt % RW) == r) {
        const size_t th = (size_t)(tb + tt) * NH + hd;
        float hsum = 0.f, nsum = 0.f;
#pragma unroll
        for (int w = 0; w < RW; ++w) {
          hsum += hpart[w][tt][lane];
          nsum += npart[w][tt];
        }
        if (has) hbuf[th * V + col] = hsum;
        if (blockIdx.z == 0 && lane == 0) {
          nq[th] = nsum;
          mt[th] = mloc[tt];
        }
      }
    }
  }
  if (has) {
#pragma unroll
    for (int d = 0; d < DQ; ++d)
      if (d0 + d < D) S[(sbase + d0 + d) * V + col] = s[d];
  }
  if (blockIdx.z == 0) {
    if (nlive) N[sbase + nd] = nn;
    if (tid == 0) M[(size_t)slot * NH + hd] = m;
  }
}

// Chunk-parallel form of the same recurrence for prompt portions (fp32 matrix cores, MFMA 16x16x4). For a chunk of
// up to 64 tokens of one row, with F_t the running sum of the log forget gates inside the chunk, b_s = i_s - F_s and
// g_t = max(m_prev, max_{s <= t} b_s)  (so that m_t = F_t + g_t, the stabiliser of the token-by-token form):
//
//   read-out_t = exp(m_prev - g_t) S_prev^T q_t + sum_{s <= t} exp(b_s - g_t) (q_t . k_s) v_s        (n . q likewise)
//   S_new      = exp(m_prev - g_L) S_prev + sum_s exp(b_s - g_L) k_s v_s^T,   m_new = F_L + g_L
//
// Every exponent is <= 0. One workgroup (four waves) per (row, head, 64 value columns) walks the row's chunks; the
// state slice S [D, 64] lives in LDS between them. Wave w owns tokens 16 w .. 16 w + 15 of the chunk for q k^T and the
// read-out, and row blocks w, w + 4, .. of S for the update. Key size up to 128.
constexpr int CL = 64;
template <typename T, int DP>
__global__ void __launch_bounds__(256) mlstm_chunk_kernel(
    const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* __restrict__ ig,
    const float* __restrict__ fg, const int* __restrict__ cu_q, const int* __restrict__ first_pos,
    const int* __restrict__ state_slots, float* __restrict__ S, float* __restrict__ N, float* __restrict__ M,
    float* __restrict__ hbuf, float* __restrict__ nq, float* __restrict__ mt, int NH, int D, int V) {
  constexpr int QS = DP + 4, CS = CL + 4;
  extern __shared__ float cl[];
  float* Sst = cl;                 // [DP][CS] state slice
  float* Qs = Sst + DP * CS;       // [CL][QS] queries / sqrt(D)
  float* Ks = Qs + CL * QS;        // [CL][QS]
  float* Vs = Ks + CL * QS;        // [CL][CS] values of this column slice
  float* Ps = Vs + CL * CS;        // [CL][CS] weighted q.k
  float* nst = Ps + CL * CS;       // [DP]
  float* Fs = nst + DP;            // [CL] running log forget
  float* bs = Fs + CL;             // [CL]
  float* gs = bs + CL;             // [CL]
  float* nqs = gs + CL;            // [CL] intra-chunk part of n . q
  float* wsl = nqs + CL;           // [CL] exp(b_s - g_L): weight of token s in the state at the chunk's end
  const int b = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, quad = lane >> 4, col0 = blockIdx.z * 64;
  const int slot = state_slots[b];
  const int t_lo = cu_q[b], t_hi = cu_q[b + 1];
  if (slot < 0) {
    for (int i = tid; i < (t_hi - t_lo) * 64; i += 256) {
      const int t = t_lo + i / 64, c = col0 + i % 64;
      if (c < V) hbuf[((size_t)t * NH + hd) * V + c] = 0.f;
      if (blockIdx.z == 0 && i % 64 == 0) nq[(size_t)t * NH + hd] = mt[(size_t)t * NH + hd] = 0.f;
    }
    return;
  }
  if (t_hi <= t_lo) return;
  const bool fresh = first_pos[b] == 0;
  const size_t sbase = ((size_t)slot * NH + hd) * D;
  for (int i = tid; i < DP * 64; i += 256) {
    const int d = i / 64, c = i % 64;
    Sst[d * CS + c] = (!fresh && d < D && col0 + c < V) ? S[(sbase + d) * V + col0 + c] : 0.f;
  }
  for (int d = tid; d < DP; d += 256) nst[d] = (!fresh && d < D) ? N[sbase + d] : 0.f;
  float m_prev = fresh ? 0.f : M[(size_t)slot * NH + hd];
  const float qscale = 1.f / sqrtf((float)D);

  for (int tb = t_lo; tb < t_hi; tb += CL) {
    const int nt = min(CL, t_hi - tb);
    __syncthreads();  // the chunk before is done with the staged operands
    if (sizeof(T) == 2 && D == DP && row_stride % 8 == 0 && k_off % 8 == 0 && q_off % 8 == 0) {  // 16-byte loads
      for (int i = tid; i < CL * DP / 8; i += 256) {
        const int d = (8 * i) % DP, tt = (8 * i) / DP;
        const bf16_t* row = reinterpret_cast<const bf16_t*>(proj) + (size_t)(tb + min(tt, nt - 1)) * row_stride;
        const bf16x8 kx = ld8(row + k_off + hd * D + d), qx = ld8(row + q_off + hd * D + d);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          Ks[tt * QS + d + e] = tt < nt ? bf2f(kx[e]) : 0.f;
          Qs[tt * QS + d + e] = tt < nt ? bf2f(qx[e]) * qscale : 0.f;
        }
      }
    } else {
      for (int i = tid; i < CL * DP; i += 256) {
        const int d = i % DP, tt = i / DP;
        const bool live = tt < nt && d < D;
        const T* row = proj + (size_t)(tb + min(tt, nt - 1)) * row_stride;
        Ks[tt * QS + d] = live ? ldf<T>(row, k_off + hd * D + d) : 0.f;
        Qs[tt * QS + d] = live ? ldf<T>(row, q_off + hd * D + d) * qscale : 0.f;
      }
    }
    for (int i = tid; i < CL * 64; i += 256) {
      const int c = i % 64, tt = i / 64;
      Vs[tt * CS + c] = (tt < nt && col0 + c < V)
                            ? ldf<T>(proj + (size_t)(tb + tt) * row_stride, v_off + hd * V + col0 + c) : 0.f;
    }
    if (w == 0) {  // running sum of f, running maximum of b = i - F, over the chunk's tokens (lane = token)
      float F = lane < nt ? fg[(size_t)(tb + lane) * NH + hd] : 0.f;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(F, o, 64);
        if (lane >= o) F += up;
      }
      const float bb = lane < nt ? ig[(size_t)(tb + lane) * NH + hd] - F : -INFINITY;
      float g = fmaxf(bb, m_prev);
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(g, o, 64);
        if (lane >= o) g = fmaxf(g, up);
      }
      Fs[lane] = F;
      bs[lane] = bb;
      gs[lane] = g;
      wsl[lane] = expf(bb - __shfl(g, 63, 64));
    }
    __syncthreads();
    // ---- P[t][s] = exp(b_s - g_t) (q_t . k_s) for s <= t; rows of wave w: t = 16 w + ..
    {
      f32x4 c[4];
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) c[cb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
      for (int kk = 0; kk < DP / 4; ++kk) {
        const float a = Qs[(16 * w + r16) * QS + 4 * kk + quad];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          if (cb <= w) c[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Ks[(16 * cb + r16) * QS + 4 * kk + quad], c[cb], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = 16 * w + 4 * quad + i;
        const float gt = gs[t];
        float rs = 0.f;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
          const int sidx = 16 * cb + r16;
          const float p = (cb <= w && sidx <= t) ? c[cb][i] * expf(bs[sidx] - gt) : 0.f;
          Ps[t * CS + sidx] = p;
          rs += p;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) rs += __shfl_xor(rs, o, 64);
        if (r16 == 0) nqs[t] = rs;
      }
    }
    __syncthreads();
    // ---- read-out of wave w's tokens: e_t (q_t S_prev) + P V; n . q
    {
      f32x4 acc[4];
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) acc[cb] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const float e_row = expf(m_prev - gs[16 * w + r16]);  // the A operand's row is token 16 w + r16
      float qn = 0.f;
#pragma unroll 4
      for (int kk = 0; kk < DP / 4; ++kk) {
        const float qv = Qs[(16 * w + r16) * QS + 4 * kk + quad];
        qn += qv * nst[4 * kk + quad];
        const float a = qv * e_row;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Sst[(4 * kk + quad) * CS + 16 * cb + r16], acc[cb], 0, 0, 0);
      }
      for (int kk = 0; kk < 4 * (w + 1); ++kk) {
        const float a = Ps[(16 * w + r16) * CS + 4 * kk + quad];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Vs[(4 * kk + quad) * CS + 16 * cb + r16], acc[cb], 0, 0, 0);
      }
      qn += __shfl_xor(qn, 16, 64);  // the four quads hold the key rows 4 kk + quad
      qn += __shfl_xor(qn, 32, 64);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int t = 16 * w + 4 * quad + i;
        if (t < nt) {
          const size_t th = (size_t)(tb + t) * NH + hd;
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) {
            const int c = col0 + 16 * cb + r16;
            if (c < V) hbuf[th * V + c] = acc[cb][i];
          }
        }
      }
      const int tq = 16 * w + r16;  // lanes of quad 0 finish n . q of token 16 w + r16
      if (blockIdx.z == 0 && quad == 0 && tq < nt) {
        const size_t th = (size_t)(tb + tq) * NH + hd;
        nq[th] = e_row * qn + nqs[tq];
        mt[th] = Fs[tq] + gs[tq];
      }
    }
    __syncthreads();  // every read of the old state is done
    // ---- state to the end of the chunk
    {
      const float gL = gs[CL - 1], decay = expf(m_prev - gL);
      for (int rb = w; rb < DP / 16; rb += 4) {
        f32x4 acc[4];
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) acc[cb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int kk = 0; kk < CL / 4; ++kk) {
          const int sidx = 4 * kk + quad;
          const float a = Ks[sidx * QS + 16 * rb + r16];
          const float ws = wsl[sidx];
#pragma unroll
          for (int cb = 0; cb < 4; ++cb)
            acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, ws * Vs[sidx * CS + 16 * cb + r16], acc[cb], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) {
            float* p = Sst + (16 * rb + 4 * quad + i) * CS + 16 * cb + r16;
            *p = decay * *p + acc[cb][i];
          }
      }
      if (tid < DP) {
        float a = decay * nst[tid];
#pragma unroll 8
        for (int sidx = 0; sidx < CL; ++sidx) a += wsl[sidx] * Ks[sidx * QS + tid];
        nst[tid] = a;
      }
      m_prev = Fs[CL - 1] + gL;
    }
  }
  __syncthreads();
  for (int i = tid; i < DP * 64; i += 256) {
    const int d = i / 64, c = i % 64;
    if (d < D && col0 + c < V) S[(sbase + d) * V + col0 + c] = Sst[d * CS + c];
  }
  if (blockIdx.z == 0) {
    for (int d = tid; d < D; d += 256) N[sbase + d] = nst[d];
    if (tid == 0) M[(size_t)slot * NH + hd] = m_prev;
  }
}

// y = h / (max(|nq|, exp(-m)) + 1e-6); per head: y / rms(y) * w * sigmoid(gate)
template <typename T>
__global__ void __launch_bounds__(256) mlstm_out_kernel(const float* __restrict__ hbuf, const float* __restrict__ nq,
                                                         const float* __restrict__ mt, const T* __restrict__ gate,
                                                         int64_t gate_stride, const T* __restrict__ w,
                                                         T* __restrict__ out, int NH, int V, float eps) {
  const size_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int hd = wave; hd < NH; hd += 4) {
    const size_t th = t * NH + hd;
    const float den = fmaxf(fabsf(nq[th]), expf(-mt[th])) + 1e-6f;
    float ss = 0.f;
    for (int v = lane; v < V; v += 64) {
      const float y = hbuf[th * V + v] / den;
      ss += y * y;
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)V + eps);
    for (int v = lane; v < V; v += 64) {
      const float y = hbuf[th * V + v] / den * r;
      const float g = ldf<T>(gate, t * gate_stride + hd * V + v);
      stf<T>(out, th * V + v, y * ldf<T>(w, hd * V + v) / (1.f + expf(-g)));
    }
  }
}

}  // namespace

extern "C" int areal_mlstm_gates(const void* x, const void* w, const void* bias, float* ig, float* fg, int T, int W,
                                 int NH, float cap, int dt, hipStream_t st) {
  if (T == 0) return 0;
  const int rows = (2 * NH + 3) / 4;
#define LAUNCH(TT, GTV)                                                                                           \
  hipLaunchKernelGGL((mlstm_gates_kernel<TT, GTV>), dim3((T + GTV - 1) / GTV, rows), dim3(256), 0, st, (const TT*)x, \
                     (const TT*)w, (const TT*)bias, ig, fg, T, W, NH, cap)
  if (dt == 0) {
    if (T < 512) LAUNCH(bf16_t, 1);
    else LAUNCH(bf16_t, 8);
  } else {
    if (T < 512) LAUNCH(float, 1);
    else LAUNCH(float, 8);
  }
#undef LAUNCH
  return (int)hipGetLastError();
}

// proj rows hold (at q_off / k_off / v_off) NH query heads of D, NH key heads of D, NH value heads of V.
// S [slots, NH, D, V], N [slots, NH, D], M [slots, NH] fp32; hbuf [T, NH, V], nq / mt [T, NH] fp32.
extern "C" int areal_mlstm_scan(const void* proj, int64_t row_stride, int q_off, int k_off, int v_off,
                                const float* ig, const float* fg, const int* cu_q, const int* first_pos,
                                const int* state_slots, float* S, float* N, float* M, float* hbuf, float* nq,
                                float* mt, int B, int NH, int D, int V, int max_q, int dt, hipStream_t st) {
  if (B == 0) return 0;
  if (D > 256 || D <= 0 || V <= 0) return -1;
  const dim3 grid(B, NH, (V + 63) / 64);
  if (max_q >= 16 && D <= 128) {  // prompt portions: the chunk-parallel kernel
#define CHUNK(TT, DPV)                                                                                             \
  do {                                                                                                             \
    const size_t lds = sizeof(float) * ((size_t)DPV * (CL + 4) + 2 * (size_t)CL * (DPV + 4) + 2 * (size_t)CL * (CL + 4) + \
                                        DPV + 5 * CL);                                                             \
    static bool raised = false;                                                                                    \
    if (!raised && lds > 64 * 1024) {                                                                              \
      HIP_RET(hipFuncSetAttribute((const void*)mlstm_chunk_kernel<TT, DPV>,                                        \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));                        \
      raised = true;                                                                                               \
    }                                                                                                              \
    hipLaunchKernelGGL((mlstm_chunk_kernel<TT, DPV>), grid, dim3(256), lds, st, (const TT*)proj, row_stride, q_off, \
                       k_off, v_off, ig, fg, cu_q, first_pos, state_slots, S, N, M, hbuf, nq, mt, NH, D, V);       \
  } while (0)
#define PICKC(TT)                      \
  do {                                 \
    if (D <= 32) CHUNK(TT, 32);        \
    else if (D <= 64) CHUNK(TT, 64);   \
    else CHUNK(TT, 128);               \
  } while (0)
    if (dt == 0) PICKC(bf16_t);
    else PICKC(float);
#undef PICKC
#undef CHUNK
    return (int)hipGetLastError();
  }
#define LAUNCH(TT, DPV)                                                                                          \
  hipLaunchKernelGGL((mlstm_scan_kernel<TT, DPV>), grid, dim3(64 * RW), 0, st, (const TT*)proj, row_stride, q_off,    \
                     k_off, v_off, ig, fg, cu_q, first_pos, state_slots, S, N, M, hbuf, nq, mt, NH, D, V)
#define PICK(TT)                 \
  do {                           \
    if (D <= 32) LAUNCH(TT, 32); \
    else if (D <= 64) LAUNCH(TT, 64); \
    else if (D <= 128) LAUNCH(TT, 128); \
    else LAUNCH(TT, 256);        \
  } while (0)
  if (dt == 0) PICK(bf16_t);
  else PICK(float);
#undef PICK
#undef LAUNCH
  return (int)hipGetLastError();
}

extern "C" int areal_mlstm_out(const float* hbuf, const float* nq, const float* mt, const void* gate,
                               int64_t gate_stride, const void* w, void* out, int T, int NH, int V, float eps, int dt,
                               hipStream_t st) {
  if (T == 0) return 0;
  if (dt == 0)
    hipLaunchKernelGGL(mlstm_out_kernel<bf16_t>, dim3(T), dim3(256), 0, st, hbuf, nq, mt, (const bf16_t*)gate,
                       gate_stride, (const bf16_t*)w, (bf16_t*)out, NH, V, eps);
  else
    hipLaunchKernelGGL(mlstm_out_kernel<float>, dim3(T), dim3(256), 0, st, hbuf, nq, mt, (const float*)gate,
                       gate_stride, (const float*)w, (float*)out, NH, V, eps);
  return (int)hipGetLastError();
}
