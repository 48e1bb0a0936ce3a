// Gated delta rule with one decay per head and key channel, over a ragged batch with per-request state slots.
//
// Per head, with S a [D, Dv] matrix kept in fp32 (stored transposed, [Dv, D], so that a column is contiguous):
//     S <- diag(decay) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// where q and k are unit vectors (q also times D^-1/2), decay = exp(-exp(a_log) * softplus(a + dt_bias)) and
// beta = sigmoid(b).  The read-out sees the token's own write.  The output is RMS-normalised over Dv, scaled by a
// weight shared by the heads and gated by sigmoid(gate).
//
// Two kernels and a small epilogue:
//   prepare  (parallel over tokens)  unit vectors q^, k^ per q/k head, decays per head and key channel, beta and
//            q^ . k^ per head, all fp32, rows padded with zeros to a multiple of 16 channels;
//   scan     every column of S evolves on its own given (q^, k^, decay, beta), so a workgroup owns one (sequence,
//            head, 16 columns) and sixteen adjacent lanes share a column, NR = D/16 rows each in registers.  The two
//            dot products of a step (k^ . dS and q^ . dS on the decayed state, o = q^ . dS + (q^ . k^) u) are summed
//            over the sixteen lanes with DPP row operations.  The prepared vectors of 32 tokens sit in LDS while
//            the next 32 are on their way from memory, so a step is one short dependent chain of register work.
//   epilogue normalises the read-out over the head's columns, applies the weight and the gate.
// The batch description is the one of the other recurrent kernels (qsl, seq_lens, slot in column 0 of the table;
// a sequence carries state in when seq_len - new_tokens > 0), so prompts, portions of prompts, single decoded
// tokens and mixtures of them are one code path, and the state after a token does not depend on how the
// sequence was cut.
#include "common.h"

__device__ __forceinline__ float dr_softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }
__device__ __forceinline__ float dr_sigmoid(float v) { return 1.f / (1.f + expf(-v)); }

// sum over the 16 lanes of a DPP row, result in every lane
__device__ __forceinline__ float row16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
  return v;
}

// grid: tokens; one wave per (token, vector): G query vectors, G key vectors (with their dot products), H decays
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    float* __restrict__ qhat, float* __restrict__ khat, float* __restrict__ dec, float* __restrict__ sc,
    const T* __restrict__ qkv, long qkv_stride, const T* __restrict__ a_raw, long a_stride,
    const T* __restrict__ b_raw, long b_stride, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    int H, int G, int D, int Dp) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float q_scale = 1.f / sqrtf((float)D);
  const int rep = H / G;
  for (int v = wave; v < G + H; v += 4) {
    if (v < G) {
      const T* qr = qkv + t * qkv_stride + (long)v * D;
      const T* kr = qkv + t * qkv_stride + (long)(G + v) * D;
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
        const float a = d < D ? (float)qr[d] * rq : 0.f, b = d < D ? (float)kr[d] * rk : 0.f;
        qhat[(t * G + v) * Dp + d] = a;
        khat[(t * G + v) * Dp + d] = b;
        dot += a * b;
      }
      dot = wave_sum(dot);
      // per head: [beta, q^ . k^]
      for (int h = v * rep + lane; h < (v + 1) * rep; h += 64) {
        sc[(t * H + h) * 2] = dr_sigmoid((float)b_raw[t * b_stride + h]);
        sc[(t * H + h) * 2 + 1] = dot;
      }
    } else {
      const int h = v - G;
      const float a_scale = expf(a_log[h]);
      for (int d = lane; d < Dp; d += 64)
        dec[(t * H + h) * Dp + d] =
            d < D ? expf(-a_scale * dr_softplus((float)a_raw[t * a_stride + (long)h * D + d] + dt_bias[(long)h * D + d]))
                  : 0.f;
    }
  }
}


// grid (heads, sequences, groups of 16 columns); block 256 = 16 columns x 16 lanes.  The prepared vectors of 32
// tokens are staged in LDS; the next 32 are on their way from memory (into registers) while these are computed.
template <typename T, int NR>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(
    float* __restrict__ o_raw, const T* __restrict__ qkv, long qkv_stride, const float* __restrict__ qhat,
    const float* __restrict__ khat, const float* __restrict__ dec, const float* __restrict__ sc,
    float* __restrict__ state, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ slot_table, long st_stride, int H, int G, int D, int Dv) {
  constexpr int Dp = 16 * NR;
  constexpr int DR_CT = NR >= 16 ? 16 : 32;            // tokens staged in LDS at a time (48 KiB at most)
  constexpr int NV = DR_CT * 16 / 256;                 // value elements a thread carries per chunk
  constexpr int VPT = DR_CT * Dp / 4;                  // float4 per staged vector kind
  constexpr int PF = (3 * VPT + 255) / 256;            // float4 a thread carries per chunk
  __shared__ __align__(16) float kqg[3 * DR_CT * Dp];  // k^ | q^ | decay, [kind][token][Dp]
  __shared__ float vv[DR_CT * 16];
  __shared__ float sc2[DR_CT * 2];
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
  const int sl = seq_lens[s];
  if (sl <= 0) return;
  const int t0 = qsl[s], L = qsl[s + 1] - t0;
  if (L <= 0) return;
  const int c = h / (H / G);
  const int col0 = blockIdx.z * 16;
  const int col = col0 + (tid >> 4), part = tid & 15;
  const bool has_col = col < Dv;
  float* Scol = state + (((long)slot_table[s * st_stride] * H + h) * Dv + (has_col ? col : Dv - 1)) * D + part * NR;
  float S[NR];
  const bool carry = sl - L > 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) S[i] = (carry && part * NR + i < D) ? Scol[i] : 0.f;

  f32x4 pre[PF];
  float pv[NV], ps = 0.f;
  auto prefetch = [&](int cs) {
    const int nt = min(DR_CT, L - cs);
#pragma unroll
    for (int n = 0; n < PF; ++n) {
      const int e = tid + n * 256;
      f32x4 x = {0.f, 0.f, 0.f, 0.f};
      if (e < 3 * VPT) {
        const int kind = e / VPT, rem = e - kind * VPT, tt = rem / (Dp / 4), j = rem - tt * (Dp / 4);
        if (tt < nt) {
          const long t = t0 + cs + tt;
          const float* src = kind == 0 ? khat + (t * G + c) * Dp : kind == 1 ? qhat + (t * G + c) * Dp
                                                                             : dec + (t * H + h) * Dp;
          x = *reinterpret_cast<const f32x4*>(src + 4 * j);
        }
      }
      pre[n] = x;
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int e = tid + n * 256, tt = e >> 4, j = e & 15;
      pv[n] = (tt < nt && col0 + j < Dv)
                  ? (float)qkv[(long)(t0 + cs + tt) * qkv_stride + (long)2 * G * D + (long)h * Dv + col0 + j] : 0.f;
    }
    if (tid < 2 * DR_CT) ps = (tid >> 1) < nt ? sc[((long)(t0 + cs + (tid >> 1)) * H + h) * 2 + (tid & 1)] : 0.f;
  };

  prefetch(0);
  for (int cs = 0; cs < L; cs += DR_CT) {
    const int nt = min(DR_CT, L - cs);
    __syncthreads();                                   // the previous chunk has been read by everybody
#pragma unroll
    for (int n = 0; n < PF; ++n) {
      const int e = tid + n * 256;
      if (e < 3 * VPT) *reinterpret_cast<f32x4*>(kqg + 4 * e) = pre[n];
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) vv[tid + n * 256] = pv[n];
    if (tid < 2 * DR_CT) sc2[tid] = ps;
    __syncthreads();
    if (cs + DR_CT < L) prefetch(cs + DR_CT);
    for (int tt = 0; tt < nt; ++tt) {
      const float* kp = kqg + tt * Dp + part * NR;
      const float* qp = kp + DR_CT * Dp;
      const float* gp = qp + DR_CT * Dp;
      float kr[NR], r = 0.f, p = 0.f;
      if constexpr (NR >= 4) {
#pragma unroll
        for (int i = 0; i < NR / 4; ++i) {
          const f32x4 k4 = reinterpret_cast<const f32x4*>(kp)[i], q4 = reinterpret_cast<const f32x4*>(qp)[i],
                      g4 = reinterpret_cast<const f32x4*>(gp)[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float sd = S[4 * i + j] * g4[j];
            S[4 * i + j] = sd;
            kr[4 * i + j] = k4[j];
            r += sd * k4[j];
            p += sd * q4[j];
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const float sd = S[i] * gp[i];
          S[i] = sd;
          kr[i] = kp[i];
          r += sd * kp[i];
          p += sd * qp[i];
        }
      }
      r = row16_sum(r);
      p = row16_sum(p);
      const float u = sc2[2 * tt] * (vv[tt * 16 + (tid >> 4)] - r);
#pragma unroll
      for (int i = 0; i < NR; ++i) S[i] += kr[i] * u;
      if (part == 0 && has_col) o_raw[(long)(t0 + cs + tt) * H * Dv + (long)h * Dv + col] = p + sc2[2 * tt + 1] * u;
    }
  }
  if (has_col) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (part * NR + i < D) Scol[i] = S[i];
  }
}

// out[t, h, :] = o / sqrt(mean(o^2) + eps) * norm_w * sigmoid(gate): one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void delta_out_norm_gate_kernel(T* __restrict__ out, long o_stride,
                                                                  const float* __restrict__ o_raw,
                                                                  const T* __restrict__ gate_raw, long g_stride,
                                                                  const float* __restrict__ norm_w, long rows, int H,
                                                                  int Dv, float eps) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);      // (token, head) pair
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const long t = row / H;
  const int h = (int)(row % H);
  const float* o = o_raw + row * Dv;
  float ss = 0.f;
  for (int j = lane; j < Dv; j += 64) ss += o[j] * o[j];
  ss = wave_sum(ss);
  const float rs = 1.f / sqrtf(ss / (float)Dv + eps);
  for (int j = lane; j < Dv; j += 64) {
    const float gt = dr_sigmoid((float)gate_raw[t * g_stride + (long)h * Dv + j]);
    out[t * o_stride + (long)h * Dv + j] = (T)(o[j] * rs * norm_w[j] * gt);
  }
}

template <typename T>
static int launch_delta_rule(int NR, dim3 grid, hipStream_t st, float* o_raw, const void* qkv, long qkv_stride,
                             const float* qhat, const float* khat, const float* dec, const float* sc, float* state,
                             const int* qsl, const int* seq_lens, const int* slot_table, long st_stride, int H, int G,
                             int D, int Dv) {
#define L(NRV)                                                                                                     \
  hipLaunchKernelGGL((gated_delta_rule_kernel<T, NRV>), grid, dim3(256), 0, st, o_raw, (const T*)qkv, qkv_stride,  \
                     qhat, khat, dec, sc, state, qsl, seq_lens, slot_table, st_stride, H, G, D, Dv)
  switch (NR) {
    case 1: L(1); break;
    case 2: L(2); break;
    case 4: L(4); break;
    case 8: L(8); break;
    case 16: L(16); break;
    default: return -2;
  }
#undef L
  return 0;
}

// channels per lane of the scan for key width D (D <= 256), and the padded row length of the prepared vectors
VDA_EXPORT int vda_delta_rule_padded_dim(int D) {
  int NR = 1;
  while (16 * NR < D) NR *= 2;
  return 16 * NR;
}

// o_raw: fp32 [T, H * Dv]; prep: fp32 scratch of T * ((2 G + H) * Dp + 2 H) floats, Dp = vda_delta_rule_padded_dim(D)
VDA_EXPORT int vda_gated_delta_rule(void* out, long o_stride, float* o_raw, float* prep, const void* qkv,
                                    long qkv_stride, const void* a_raw, long a_stride, const void* b_raw,
                                    long b_stride, const void* gate_raw, long g_stride, const float* a_log,
                                    const float* dt_bias, const float* norm_w, float* state, const int* qsl,
                                    const int* seq_lens, const int* slot_table, long st_stride, int T_tokens, int S,
                                    int H, int G, int D, int Dv, float eps, int dtype, hipStream_t st) {
  if (S <= 0 || T_tokens <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D < 1 || D > 256 || Dv < 1) return -1;
  const int Dp = vda_delta_rule_padded_dim(D), NR = Dp / 16;
  float* qhat = prep;
  float* khat = qhat + (size_t)T_tokens * G * Dp;
  float* dec = khat + (size_t)T_tokens * G * Dp;
  float* sc = dec + (size_t)T_tokens * H * Dp;
#define LP(TT) hipLaunchKernelGGL((delta_prepare_kernel<TT>), dim3(T_tokens), dim3(256), 0, st, qhat, khat, dec, sc, \
                                  (const TT*)qkv, qkv_stride, (const TT*)a_raw, a_stride, (const TT*)b_raw, b_stride, \
                                  a_log, dt_bias, H, G, D, Dp)
  if (dtype == VDA_BF16) LP(bf16_t);
  else if (dtype == VDA_F16) LP(f16_t);
  else if (dtype == VDA_F32) LP(float);
  else return -3;
#undef LP
  VDA_CHECK_LAUNCH();
  dim3 grid(H, S, (Dv + 15) / 16);
  int rc;
  if (dtype == VDA_BF16)
    rc = launch_delta_rule<bf16_t>(NR, grid, st, o_raw, qkv, qkv_stride, qhat, khat, dec, sc, state, qsl, seq_lens,
                                   slot_table, st_stride, H, G, D, Dv);
  else if (dtype == VDA_F16)
    rc = launch_delta_rule<f16_t>(NR, grid, st, o_raw, qkv, qkv_stride, qhat, khat, dec, sc, state, qsl, seq_lens,
                                  slot_table, st_stride, H, G, D, Dv);
  else
    rc = launch_delta_rule<float>(NR, grid, st, o_raw, qkv, qkv_stride, qhat, khat, dec, sc, state, qsl, seq_lens,
                                  slot_table, st_stride, H, G, D, Dv);
  if (rc) return rc;
  VDA_CHECK_LAUNCH();
  const long rows = (long)T_tokens * H;
  dim3 g2((unsigned)((rows + 3) / 4)), b2(256);
#define L2(TT) hipLaunchKernelGGL((delta_out_norm_gate_kernel<TT>), g2, b2, 0, st, (TT*)out, o_stride, o_raw, \
                                  (const TT*)gate_raw, g_stride, norm_w, rows, H, Dv, eps)
  if (dtype == VDA_BF16) L2(bf16_t);
  else if (dtype == VDA_F16) L2(f16_t);
  else L2(float);
#undef L2
  VDA_CHECK_LAUNCH();
  return 0;
}
