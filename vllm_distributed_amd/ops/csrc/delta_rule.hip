// Gated delta rule with one decay per head and key channel, over a ragged batch with per-request state slots.
//
// Per head, with S a [D, Dv] matrix kept in fp32 (stored transposed, [Dv, D], so that a column is contiguous):
//     S <- diag(decay) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// where q and k are unit vectors (q also times D^-1/2), decay = exp(-exp(a_log) * softplus(a + dt_bias)) and
// beta = sigmoid(b).  The read-out sees the token's own write.  The output is RMS-normalised over Dv, scaled by a
// weight shared by the heads and gated by sigmoid(gate).
//
// Every column of S evolves on its own given (q, k, decay, beta), so a workgroup owns one (sequence, head, group of
// 32 columns) and its threads own columns: four adjacent lanes share a column, NR = D/4 rows each in registers, and
// the two dot products of a step (k . dS and q . dS, taken on the decayed state before the write, o = q . dS +
// (q . k) u) are summed over the four lanes together.  Tokens are walked in chunks of 16: the chunk's unit vectors,
// decays and gates are computed once by all threads (fp32) into LDS -- all loads of a chunk issued together, rows
// padded so that the four lanes of a column read different banks with 16-byte loads -- then every thread runs its
// column through the chunk.  The read-out goes
// to an fp32 scratch; a second small kernel normalises it over the head's columns and gates it.
// The batch description is the one of the other recurrent kernels (qsl, seq_lens, slot in column 0 of the table;
// a sequence carries state in when seq_len - new_tokens > 0), so prompts, portions of prompts, single decoded
// tokens and mixtures of them are one code path, and the state after a token does not depend on how the
// sequence was cut.
#include "common.h"

#define DR_CT 16

__device__ __forceinline__ float dr_softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }
__device__ __forceinline__ float dr_sigmoid(float v) { return 1.f / (1.f + expf(-v)); }

// LDS row of one token's vector: the four row groups (one per lane of a column) sit NR + pad floats apart so that
// their 16-byte reads fall into different banks
template <int NR> struct DrRow {
  static constexpr int PS = NR + (NR == 12 ? 8 : 4);
  static constexpr int LEN = 4 * PS;
};

// grid (heads, sequences, column groups); block 4 * Cw threads, Cw columns of S per workgroup.  Writes the raw
// read-out o (fp32) to `o_raw` [T, H * Dv]; vda_gated_delta_rule's second kernel normalises and gates it.
template <typename T, int NR>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(
    float* __restrict__ o_raw, const T* __restrict__ qkv, long qkv_stride, const T* __restrict__ a_raw,
    long a_stride, const T* __restrict__ b_raw, long b_stride, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, const int* __restrict__ slot_table, long st_stride, int H, int G, int D,
    int Dv, int Cw) {
  constexpr int PS = DrRow<NR>::PS, RL = DrRow<NR>::LEN;
  extern __shared__ __align__(16) float lds[];
  const int nthreads = blockDim.x;
  float* qh = lds;                      // [CT][RL]
  float* kh = qh + DR_CT * RL;          // [CT][RL]
  float* gh = kh + DR_CT * RL;          // [CT][RL]
  float* vv = gh + DR_CT * RL;          // [CT][Cw]
  float* qk = vv + DR_CT * Cw;          // [CT]
  float* bt = qk + DR_CT;               // [CT]

  const int h = blockIdx.x, s = blockIdx.y, col0 = blockIdx.z * Cw, tid = threadIdx.x;
  const int sl = seq_lens[s];
  if (sl <= 0) return;
  const int t0 = qsl[s], L = qsl[s + 1] - t0;
  if (L <= 0) return;
  const int c = h / (H / G);            // q / k head of this head
  const int col = col0 + (tid >> 2), part = tid & 3;
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
    // ---- the chunk's inputs: every thread loads its share at once (one trip to memory per chunk) ------------
    for (int e = tid; e < nt * D; e += nthreads) {
      const int tt = e / D, d = e - tt * D;
      const long t = t0 + cs + tt;
      const int at = tt * RL + (d / NR) * PS + d % NR;
      qh[at] = (float)qkv[t * qkv_stride + (long)c * D + d];
      kh[at] = (float)qkv[t * qkv_stride + (long)(G + c) * D + d];
      gh[at] = (float)a_raw[t * a_stride + (long)h * D + d];
    }
    for (int e = tid; e < nt * Cw; e += nthreads) {
      const int tt = e / Cw, j = e - tt * Cw;
      vv[e] = col0 + j < Dv ? (float)qkv[(long)(t0 + cs + tt) * qkv_stride + (long)2 * G * D + (long)h * Dv + col0 + j]
                            : 0.f;
    }
    if (tid < nt) bt[tid] = dr_sigmoid((float)b_raw[(long)(t0 + cs + tid) * b_stride + h]);
    __syncthreads();
    // ---- unit vectors and decays in place, one wave per token ---------------------------------------------------
    for (int tt = wave; tt < nt; tt += nw) {
      float sq = 0.f, sk = 0.f;
      for (int d = lane; d < D; d += 64) {
        const int at = tt * RL + (d / NR) * PS + d % NR;
        const float a = qh[at], b = kh[at];
        sq += a * a;
        sk += b * b;
      }
      sq = wave_sum(sq);
      sk = wave_sum(sk);
      const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.f / sqrtf(sk + 1e-6f);
      float dot = 0.f;
      for (int d = lane; d < 4 * NR; d += 64) {
        const int at = tt * RL + (d / NR) * PS + d % NR;
        float a = 0.f, b = 0.f, g = 0.f;
        if (d < D) {
          a = qh[at] * rq;
          b = kh[at] * rk;
          g = expf(-a_scale * dr_softplus(gh[at] + dt_bias[(long)h * D + d]));
        }
        qh[at] = a;
        kh[at] = b;
        gh[at] = g;
        dot += a * b;
      }
      dot = wave_sum(dot);
      if (lane == 0) qk[tt] = dot;
    }
    __syncthreads();
    // ---- the recurrence: every thread its rows of one column ------------------------------------------------
    for (int tt = 0; tt < nt; ++tt) {
      const f32x4* kp = reinterpret_cast<const f32x4*>(kh + tt * RL + part * PS);
      const f32x4* qp = reinterpret_cast<const f32x4*>(qh + tt * RL + part * PS);
      const f32x4* gp = reinterpret_cast<const f32x4*>(gh + tt * RL + part * PS);
      f32x4 kreg[NR / 4];
      float r0 = 0.f, r1 = 0.f, p0 = 0.f, p1 = 0.f;
#pragma unroll
      for (int i = 0; i < NR / 4; ++i) {
        const f32x4 g4 = gp[i], k4 = kp[i], q4 = qp[i];
        kreg[i] = k4;
        const float s0 = S[4 * i] * g4[0], s1 = S[4 * i + 1] * g4[1], s2 = S[4 * i + 2] * g4[2],
                    s3 = S[4 * i + 3] * g4[3];
        S[4 * i] = s0;
        S[4 * i + 1] = s1;
        S[4 * i + 2] = s2;
        S[4 * i + 3] = s3;
        r0 += s0 * k4[0] + s2 * k4[2];
        r1 += s1 * k4[1] + s3 * k4[3];
        p0 += s0 * q4[0] + s2 * q4[2];
        p1 += s1 * q4[1] + s3 * q4[3];
      }
      float r = r0 + r1, p = p0 + p1;
      r += __shfl_xor(r, 1, 64);
      p += __shfl_xor(p, 1, 64);
      r += __shfl_xor(r, 2, 64);
      p += __shfl_xor(p, 2, 64);
      const float u = bt[tt] * (vv[tt * Cw + (tid >> 2)] - r);
#pragma unroll
      for (int i = 0; i < NR / 4; ++i) {
        S[4 * i] += kreg[i][0] * u;
        S[4 * i + 1] += kreg[i][1] * u;
        S[4 * i + 2] += kreg[i][2] * u;
        S[4 * i + 3] += kreg[i][3] * u;
      }
      if (part == 0 && has_col) o_raw[(long)(t0 + cs + tt) * H * Dv + (long)h * Dv + col] = p + qk[tt] * u;
    }
    __syncthreads();
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
static int launch_delta_rule(int NRsel, dim3 grid, dim3 block, hipStream_t st, float* o_raw, const void* qkv,
                             long qkv_stride, const void* a_raw, long a_stride, const void* b_raw, long b_stride,
                             const float* a_log, const float* dt_bias, float* state, const int* qsl,
                             const int* seq_lens, const int* slot_table, long st_stride, int H, int G, int D, int Dv,
                             int Cw) {
#define L(NRV)                                                                                                        \
  do {                                                                                                                \
    const size_t lds = ((size_t)DR_CT * (3 * DrRow<NRV>::LEN + Cw) + 2 * DR_CT) * sizeof(float);                      \
    if (lds > 48 * 1024) {                                                                                            \
      hipError_t e = hipFuncSetAttribute((const void*)gated_delta_rule_kernel<T, NRV>,                               \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                       \
      if (e != hipSuccess) return (int)e;                                                                             \
    }                                                                                                                 \
    hipLaunchKernelGGL((gated_delta_rule_kernel<T, NRV>), grid, block, lds, st, o_raw, (const T*)qkv, qkv_stride,     \
                       (const T*)a_raw, a_stride, (const T*)b_raw, b_stride, a_log, dt_bias, state, qsl, seq_lens,    \
                       slot_table, st_stride, H, G, D, Dv, Cw);                                                       \
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

// o_raw: fp32 scratch [T, H * Dv] of the caller
VDA_EXPORT int vda_gated_delta_rule(void* out, long o_stride, float* o_raw, const void* qkv, long qkv_stride,
                                    const void* a_raw, long a_stride, const void* b_raw, long b_stride,
                                    const void* gate_raw, long g_stride, const float* a_log, const float* dt_bias,
                                    const float* norm_w, float* state, const int* qsl, const int* seq_lens,
                                    const int* slot_table, long st_stride, int T_tokens, int S, int H, int G, int D,
                                    int Dv, float eps, int dtype, hipStream_t st) {
  if (S <= 0 || T_tokens <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D < 1 || D > 256 || Dv < 1) return -1;
  static const int sizes[] = {4, 8, 12, 16, 24, 32, 48, 64};
  int NR = 0;
  for (int v : sizes)
    if (4 * v >= D) { NR = v; break; }
  // columns per workgroup: 32 (two waves) unless the head is narrower; wide rows keep 16 to stay within registers
  int Cw = NR > 32 ? 16 : 32;
  if (Dv <= 16) Cw = 16;
  dim3 grid(H, S, (Dv + Cw - 1) / Cw), block(4 * Cw);
  int rc;
  if (dtype == VDA_BF16)
    rc = launch_delta_rule<bf16_t>(NR, grid, block, st, o_raw, qkv, qkv_stride, a_raw, a_stride, b_raw, b_stride,
                                   a_log, dt_bias, state, qsl, seq_lens, slot_table, st_stride, H, G, D, Dv, Cw);
  else if (dtype == VDA_F16)
    rc = launch_delta_rule<f16_t>(NR, grid, block, st, o_raw, qkv, qkv_stride, a_raw, a_stride, b_raw, b_stride,
                                  a_log, dt_bias, state, qsl, seq_lens, slot_table, st_stride, H, G, D, Dv, Cw);
  else if (dtype == VDA_F32)
    rc = launch_delta_rule<float>(NR, grid, block, st, o_raw, qkv, qkv_stride, a_raw, a_stride, b_raw, b_stride,
                                  a_log, dt_bias, state, qsl, seq_lens, slot_table, st_stride, H, G, D, Dv, Cw);
  else
    return -3;
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
