// Gated delta rule with one decay per head and key channel, over a ragged batch with per-request state slots.
//
// Per head, with S a [D, Dv] matrix kept in fp32 (stored transposed, [Dv, D], so that a column is contiguous):
//     S <- diag(decay) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// where q and k are unit vectors (q also times D^-1/2), decay = exp(-exp(a_log) * softplus(a + dt_bias)) and
// beta = sigmoid(b).  The read-out sees the token's own write.  The output is RMS-normalised over Dv, scaled by a
// weight shared by the heads and gated by sigmoid(gate).
//
// Every column of S evolves on its own given (q, k, decay, beta), so a workgroup owns one (sequence, head) and its
// threads own columns: four adjacent lanes share a column, NR = D/4 rows each in registers, and the two dot
// products of a step (k . dS and q . dS, taken on the decayed state before the write, o = q . dS + (q . k) u) are
// summed over the four lanes together.  Tokens are walked in chunks of 16: the chunk's unit vectors, decays and
// gates are computed once by all threads (fp32) into LDS, then every thread runs its columns through the chunk.
// The batch description is the one of the other recurrent kernels (qsl, seq_lens, slot in column 0 of the table;
// a sequence carries state in when seq_len - new_tokens > 0), so prompts, portions of prompts, single decoded
// tokens and mixtures of them are one code path, and the state after a token does not depend on how the
// sequence was cut.
#include "common.h"

#define DR_CT 16

__device__ __forceinline__ float dr_softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }
__device__ __forceinline__ float dr_sigmoid(float v) { return 1.f / (1.f + expf(-v)); }

template <typename T, int NR>
__global__ __launch_bounds__(1024) void gated_delta_rule_kernel(
    T* __restrict__ out, long o_stride, const T* __restrict__ qkv, long qkv_stride, const T* __restrict__ a_raw,
    long a_stride, const T* __restrict__ b_raw, long b_stride, const T* __restrict__ gate_raw, long g_stride,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ norm_w,
    float* __restrict__ state, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ slot_table, long st_stride, int H, int G, int D, int Dv, float eps) {
  constexpr int Dp = 4 * NR;
  extern __shared__ float lds[];
  const int nthreads = blockDim.x, Cw = nthreads >> 2;
  float* qh = lds;                      // [CT][Dp]
  float* kh = qh + DR_CT * Dp;          // [CT][Dp]
  float* gh = kh + DR_CT * Dp;          // [CT][Dp]
  float* vv = gh + DR_CT * Dp;          // [CT][Cw]
  float* ob = vv + DR_CT * Cw;          // [CT][Cw]
  float* qk = ob + DR_CT * Cw;          // [CT]
  float* bt = qk + DR_CT;               // [CT]

  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
  const int sl = seq_lens[s];
  if (sl <= 0) return;
  const int t0 = qsl[s], L = qsl[s + 1] - t0;
  if (L <= 0) return;
  const int c = h / (H / G);            // q / k head of this head
  const int col = tid >> 2, part = tid & 3;
  const int lane = tid & 63, wave = tid >> 6, nw = nthreads >> 6;
  const bool has_col = col < Dv;
  float* Scol = state + (((long)slot_table[s * st_stride] * H + h) * Dv + (has_col ? col : 0)) * D + part * NR;
  float S[NR];
  const bool carry = sl - L > 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) S[i] = (carry && has_col && part * NR + i < D) ? Scol[i] : 0.f;
  const float a_scale = expf(a_log[h]);
  const float q_scale = 1.f / sqrtf((float)D);

  for (int cs = 0; cs < L; cs += DR_CT) {
    const int nt = min(DR_CT, L - cs);
    // ---- the chunk's vectors, by all threads: one wave per token -----------------------------------------
    for (int tt = wave; tt < nt; tt += nw) {
      const long t = t0 + cs + tt;
      const T* qr = qkv + t * qkv_stride + (long)c * D;
      const T* kr = qkv + t * qkv_stride + (long)(G + c) * D;
      float sq = 0.f, sk = 0.f;
      for (int d = lane; d < D; d += 64) {
        const float a = (float)qr[d], b = (float)kr[d];
        sq += a * a;
        sk += b * b;
      }
      sq = wave_sum(sq);
      sk = wave_sum(sk);
      const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.f / sqrtf(sk + 1e-6f);
      float dot = 0.f;
      for (int d = lane; d < Dp; d += 64) {
        float a = 0.f, b = 0.f, g = 0.f;
        if (d < D) {
          a = (float)qr[d] * rq;
          b = (float)kr[d] * rk;
          g = expf(-a_scale * dr_softplus((float)a_raw[t * a_stride + (long)h * D + d] + dt_bias[(long)h * D + d]));
        }
        qh[tt * Dp + d] = a;
        kh[tt * Dp + d] = b;
        gh[tt * Dp + d] = g;
        dot += a * b;
      }
      dot = wave_sum(dot);
      if (lane == 0) {
        qk[tt] = dot;
        bt[tt] = dr_sigmoid((float)b_raw[t * b_stride + h]);
      }
      for (int j = lane; j < Cw; j += 64)
        vv[tt * Cw + j] = j < Dv ? (float)qkv[t * qkv_stride + (long)2 * G * D + (long)h * Dv + j] : 0.f;
    }
    __syncthreads();
    // ---- the recurrence: every thread its rows of one column ------------------------------------------------
    for (int tt = 0; tt < nt; ++tt) {
      const float* kp = kh + tt * Dp + part * NR;
      const float* qp = qh + tt * Dp + part * NR;
      const float* gp = gh + tt * Dp + part * NR;
      float r = 0.f, p = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const float sd = S[i] * gp[i];
        S[i] = sd;
        r += sd * kp[i];
        p += sd * qp[i];
      }
      r += __shfl_xor(r, 1, 64);
      p += __shfl_xor(p, 1, 64);
      r += __shfl_xor(r, 2, 64);
      p += __shfl_xor(p, 2, 64);
      const float u = bt[tt] * (vv[tt * Cw + col] - r);
#pragma unroll
      for (int i = 0; i < NR; ++i) S[i] += kp[i] * u;
      if (part == 0) ob[tt * Cw + col] = p + qk[tt] * u;
    }
    __syncthreads();
    // ---- output: RMS over the head's Dv values, weight, gate ----------------------------------------------
    for (int tt = wave; tt < nt; tt += nw) {
      const long t = t0 + cs + tt;
      float ss = 0.f;
      for (int j = lane; j < Dv; j += 64) {
        const float o = ob[tt * Cw + j];
        ss += o * o;
      }
      ss = wave_sum(ss);
      const float rs = 1.f / sqrtf(ss / (float)Dv + eps);
      for (int j = lane; j < Dv; j += 64) {
        const float gt = dr_sigmoid((float)gate_raw[t * g_stride + (long)h * Dv + j]);
        out[t * o_stride + (long)h * Dv + j] = (T)(ob[tt * Cw + j] * rs * norm_w[j] * gt);
      }
    }
    __syncthreads();
  }
  if (has_col) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (part * NR + i < D) Scol[i] = S[i];
  }
}

template <typename T>
static int launch_delta_rule(int NRsel, dim3 grid, dim3 block, size_t lds, hipStream_t st, void* out, long o_stride,
                             const void* qkv, long qkv_stride, const void* a_raw, long a_stride, const void* b_raw,
                             long b_stride, const void* gate_raw, long g_stride, const float* a_log,
                             const float* dt_bias, const float* norm_w, float* state, const int* qsl,
                             const int* seq_lens, const int* slot_table, long st_stride, int H, int G, int D, int Dv,
                             float eps) {
#define L(NRV)                                                                                                        \
  do {                                                                                                                \
    if (lds > 48 * 1024) {                                                                                            \
      hipError_t e = hipFuncSetAttribute((const void*)gated_delta_rule_kernel<T, NRV>,                               \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                       \
      if (e != hipSuccess) return (int)e;                                                                             \
    }                                                                                                                 \
    hipLaunchKernelGGL((gated_delta_rule_kernel<T, NRV>), grid, block, lds, st, (T*)out, o_stride, (const T*)qkv,     \
                       qkv_stride, (const T*)a_raw, a_stride, (const T*)b_raw, b_stride, (const T*)gate_raw, g_stride, \
                       a_log, dt_bias, norm_w, state, qsl, seq_lens, slot_table, st_stride, H, G, D, Dv, eps);        \
  } while (0)
  switch (NRsel) {
    case 4: L(4); break;
    case 8: L(8); break;
    case 12: L(12); break;
    case 16: L(16); break;
    case 24: L(24); break;
    case 32: L(32); break;
    case 48: L(48); break;
    case 64: L(64); break;
    default: return -2;
  }
#undef L
  return 0;
}

VDA_EXPORT int vda_gated_delta_rule(void* out, long o_stride, const void* qkv, long qkv_stride, const void* a_raw,
                                    long a_stride, const void* b_raw, long b_stride, const void* gate_raw,
                                    long g_stride, const float* a_log, const float* dt_bias, const float* norm_w,
                                    float* state, const int* qsl, const int* seq_lens, const int* slot_table,
                                    long st_stride, int S, int H, int G, int D, int Dv, float eps, int dtype,
                                    hipStream_t st) {
  if (S <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D < 1 || D > 256 || Dv < 1 || Dv > 256) return -1;
  static const int sizes[] = {4, 8, 12, 16, 24, 32, 48, 64};
  int NR = 0;
  for (int v : sizes)
    if (4 * v >= D) { NR = v; break; }
  const int Cw = (Dv + 15) / 16 * 16;
  dim3 grid(H, S), block(4 * Cw);
  const size_t lds = ((size_t)DR_CT * (3 * 4 * NR + 2 * Cw) + 2 * DR_CT) * sizeof(float);
  int rc;
  if (dtype == VDA_BF16)
    rc = launch_delta_rule<bf16_t>(NR, grid, block, lds, st, out, o_stride, qkv, qkv_stride, a_raw, a_stride, b_raw,
                                   b_stride, gate_raw, g_stride, a_log, dt_bias, norm_w, state, qsl, seq_lens,
                                   slot_table, st_stride, H, G, D, Dv, eps);
  else if (dtype == VDA_F16)
    rc = launch_delta_rule<f16_t>(NR, grid, block, lds, st, out, o_stride, qkv, qkv_stride, a_raw, a_stride, b_raw,
                                  b_stride, gate_raw, g_stride, a_log, dt_bias, norm_w, state, qsl, seq_lens,
                                  slot_table, st_stride, H, G, D, Dv, eps);
  else if (dtype == VDA_F32)
    rc = launch_delta_rule<float>(NR, grid, block, lds, st, out, o_stride, qkv, qkv_stride, a_raw, a_stride, b_raw,
                                  b_stride, gate_raw, g_stride, a_log, dt_bias, norm_w, state, qsl, seq_lens,
                                  slot_table, st_stride, H, G, D, Dv, eps);
  else
    return -3;
  if (rc) return rc;
  VDA_CHECK_LAUNCH();
  return 0;
}
