// Matrix memory with exponential gates and a running maximum (the mLSTM cell of xLSTM), over a ragged batch with a
// carried fp32 state per request.
//
// Per token and head, with q scaled by D^-1/2 and the gate pre-activations i_raw, f_raw:
//   i = cap * tanh((i_raw + i_bias) / cap)          f = logsigmoid(cap * tanh((f_raw + f_bias) / cap))
//   m' = max(f + m, i)        a = exp(f + m - m')   b = exp(i - m')
//   S' = a S + b k v^T        n' = a n + b k        (S: [D, Dv], n: [D];  m, S, n start at zero)
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// followed, in a second launch, by out = o / rms(o) per head * weight * sigmoid(output gate).
//
// The scan: one workgroup per (sequence, head, group of value columns).  A column's D state values are spread over
// LPC lanes (DPT values each, in registers); every lane also carries its part of n, so S'^T q and n' . q are two
// partial sums reduced over the LPC lanes by shuffles.  q, k, v and the gates of 16 tokens at a time are staged
// through LDS; the max / exp recurrence is a few scalar operations that every lane repeats.  Tokens are walked one
// by one from the carried state, so results do not depend on how a prompt is cut.
#include "common.h"

#define MLSTM_TCH_MAX 16          // tokens staged through LDS at a time (fewer for very wide heads)

__device__ __forceinline__ float logsigmoid_f(float x) {
  // -softplus(-x), stable for both signs
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

template <typename T, int DPT>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(
    float* __restrict__ o_raw, const T* __restrict__ proj, long p_stride, const float* __restrict__ i_bias,
    const float* __restrict__ f_bias, float* __restrict__ state_nm, float* __restrict__ state_s,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens, const int* __restrict__ slot_table,
    long st_stride, int H, int D, int Dv, int Dn, int LPC, int TCH, float cap) {
  extern __shared__ float lds[];
  const int DP = LPC * DPT;                       // D rounded up; the tail stays zero
  const int CW = 256 / LPC;                       // value columns of this workgroup
  float* qs = lds;                                // [TCH][DP]
  float* ks = qs + TCH * DP;                      // [TCH][DP]
  float* vs = ks + TCH * DP;                      // [TCH][CW]
  float* gi = vs + TCH * CW;                      // [TCH]
  float* gf = gi + TCH;                           // [TCH]

  const int s = blockIdx.z, h = blockIdx.y, tid = threadIdx.x;
  const int sl = seq_lens[s];
  if (sl <= 0) return;
  const int t0 = qsl[s], L = qsl[s + 1] - t0;
  if (L <= 0) return;
  const bool has_init = sl - L > 0;
  const int part = tid % LPC, col = blockIdx.x * CW + tid / LPC;
  const bool live = col < Dv;
  const long slot = slot_table[(long)s * st_stride];
  float* sp = state_s + ((slot * H + h) * D) * (long)Dv + col;
  float* np = state_nm + (slot * H + h) * (long)Dn;
  const int d0 = part * DPT;
  float S[DPT], n[DPT];
  float m = 0.f;
#pragma unroll
  for (int dd = 0; dd < DPT; ++dd) {
    const int d = d0 + dd;
    const bool ok = has_init && d < D;
    S[dd] = ok && live ? sp[(long)d * Dv] : 0.f;
    n[dd] = ok ? np[d] : 0.f;
  }
  if (has_init) m = np[D];
  const float qscale = rsqrtf((float)D);
  const int HD = H * D, HV = H * Dv;
  const T* pq = proj + (long)h * D;
  const T* pk = proj + HD + (long)h * D;
  const T* pv = proj + 2 * HD + (long)h * Dv + blockIdx.x * CW;
  const T* pi = proj + 2 * HD + 2 * HV + h;
  const T* pf = pi + H;
  const float bi = i_bias[h], bf = f_bias[h];

  for (int c0 = 0; c0 < L; c0 += TCH) {
    const int nt = min(TCH, L - c0);
    __syncthreads();
    for (int e = tid; e < TCH * DP; e += 256) {
      const int d = e % DP, tt = e / DP;
      float qv = 0.f, kv = 0.f;
      if (tt < nt && d < D) {
        const long r = (long)(t0 + c0 + tt) * p_stride;
        qv = (float)pq[r + d] * qscale;
        kv = (float)pk[r + d];
      }
      qs[e] = qv;
      ks[e] = kv;
    }
    for (int e = tid; e < TCH * CW; e += 256) {
      const int c = e % CW, tt = e / CW;
      vs[e] = (tt < nt && blockIdx.x * CW + c < Dv) ? (float)pv[(long)(t0 + c0 + tt) * p_stride + c] : 0.f;
    }
    if (tid < nt) {
      const long r = (long)(t0 + c0 + tid) * p_stride;
      gi[tid] = cap * tanhf(((float)pi[r] + bi) / cap);
      gf[tid] = logsigmoid_f(cap * tanhf(((float)pf[r] + bf) / cap));
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float ig = gi[tt], fg = gf[tt];
      const float m2 = fmaxf(fg + m, ig);
      const float a = expf(fg + m - m2), b = expf(ig - m2);
      m = m2;
      const float bv = b * vs[tt * CW + tid / LPC];
      const float* qp = qs + tt * DP + d0;
      const float* kp = ks + tt * DP + d0;
      float num = 0.f, nq = 0.f;
#pragma unroll
      for (int dd = 0; dd < DPT; ++dd) {
        const float kd = kp[dd], qd = qp[dd];
        S[dd] = a * S[dd] + kd * bv;
        n[dd] = a * n[dd] + b * kd;
        num += S[dd] * qd;
        nq += n[dd] * qd;
      }
      for (int o = LPC >> 1; o > 0; o >>= 1) {
        num += __shfl_xor(num, o, 64);
        nq += __shfl_xor(nq, o, 64);
      }
      if (part == 0 && live) {
        const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
        o_raw[(long)(t0 + c0 + tt) * HV + (long)h * Dv + col] = num / den;
      }
    }
  }
#pragma unroll
  for (int dd = 0; dd < DPT; ++dd) {
    const int d = d0 + dd;
    if (d < D) {
      if (live) sp[(long)d * Dv] = S[dd];
      if (blockIdx.x == 0 && tid < LPC) np[d] = n[dd];
    }
  }
  if (blockIdx.x == 0 && tid == 0) np[D] = m;
}

// out[t, h, :] = o / rms(o) * weight[h, :] * sigmoid(gate[t, h, :]); one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(64) void mlstm_out_kernel(T* __restrict__ out, long o_stride,
                                                       const float* __restrict__ o_raw, const T* __restrict__ gate,
                                                       long g_stride, const float* __restrict__ weight, int H, int Dv,
                                                       float eps) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* op = o_raw + (t * H + h) * Dv;
  float ss = 0.f;
  for (int c = lane; c < Dv; c += 64) ss += op[c] * op[c];
  ss = wave_sum(ss);
  const float r = 1.f / sqrtf(ss / (float)Dv + eps);
  for (int c = lane; c < Dv; c += 64) {
    const float g = (float)gate[t * g_stride + (long)h * Dv + c];
    out[t * o_stride + (long)h * Dv + c] = (T)(op[c] * r * weight[h * Dv + c] / (1.f + expf(-g)));
  }
}

VDA_EXPORT int vda_mlstm(void* out, long o_stride, float* o_raw, const void* proj, long p_stride, const float* i_bias,
                         const float* f_bias, const float* weight, float* state_nm, float* state_s, const int* qsl,
                         const int* seq_lens, const int* slot_table, long st_stride, int T, int S, int H, int D,
                         int Dv, int Dn, float cap, float eps, int dtype, hipStream_t st) {
  if (T <= 0 || S <= 0) return 0;
  if (H <= 0 || D <= 0 || Dv <= 0 || Dn < D + 1) return -1;
  int LPC = 1;
  while ((D + LPC - 1) / LPC > 16 && LPC < 64) LPC <<= 1;      // 16 state values per lane: short steps, many lanes
  const int per = (D + LPC - 1) / LPC;
  if (per > 32) return -2;                       // D beyond 2048
  const int DPT = per <= 8 ? 8 : per <= 16 ? 16 : 32;
  const int CW = 256 / LPC;
  int TCH = MLSTM_TCH_MAX;
  auto lds_of = [&](int tch) { return ((size_t)2 * tch * LPC * DPT + (size_t)tch * CW + 2 * tch) * 4; };
  while (TCH > 1 && lds_of(TCH) > 60 * 1024) TCH >>= 1;
  const size_t lds = lds_of(TCH);
  dim3 grid((Dv + CW - 1) / CW, H, S), block(256);
  const long gate_off = 2L * H * D + (long)H * Dv;
#define L2(TT, DD)                                                                                                   \
  do {                                                                                                               \
    if (lds > 48 * 1024) {                                                                                           \
      hipError_t e = hipFuncSetAttribute((const void*)mlstm_scan_kernel<TT, DD>,                                     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                      \
      if (e != hipSuccess) return (int)e;                                                                            \
    }                                                                                                                \
    hipLaunchKernelGGL((mlstm_scan_kernel<TT, DD>), grid, block, lds, st, o_raw, (const TT*)proj, p_stride, i_bias,  \
                       f_bias, state_nm, state_s, qsl, seq_lens, slot_table, st_stride, H, D, Dv, Dn, LPC, TCH, cap);     \
    hipLaunchKernelGGL((mlstm_out_kernel<TT>), dim3(T, H), dim3(64), 0, st, (TT*)out, o_stride, o_raw,               \
                       (const TT*)proj + gate_off, p_stride, weight, H, Dv, eps);                                    \
  } while (0)
#define L(TT) do { if (DPT == 8) L2(TT, 8); else if (DPT == 16) L2(TT, 16); else L2(TT, 32); } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
  VDA_CHECK_LAUNCH();
  return 0;
}
