// Sigmoid attention with mixed head scores ("talking heads" before the weight function), over a sliding window
// plus the first tokens of the sequence, on the paged cache.  No softmax: nothing is normalised over keys.
//
//   raw[g](i, j)  = scale * qn[i, g] . kn[j, kv(g)]          qn, kn: per-head RMS-normalised, no learned weight
//   s[h](i, j)    = sum_g talk[h, g] raw[g](i, j) + pb[h]
//   out[i, h]     = sum over visible j of sigmoid(s[h](i, j)) * v[j, kv(h)]
//   visible: j <= i and (i - j < window or j < keep_first); window == 0: every j <= i
//
// Cache layout of this layer kind: k_cache [blocks, G, block_size, D], v_cache [blocks, G, block_size, Dv].
//
//   vda_unit_rms_qk_cache         q -> qn (fp32 [T, H, D]); kn and v -> cache at slot_mapping
//   vda_sigmoid_window_attention  one workgroup per (sequence, tile of BQ query tokens); scores, mixing and the
//                                 weight function in fp32; keys outside the window and the kept prefix are never
//                                 loaded.  Prompts, portions of prompts and single decoded tokens are one code path.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void unit_rms_qk_cache_kernel(
    float* __restrict__ qn, const T* __restrict__ qkv, long qkv_stride, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const long* __restrict__ slot_mapping, int H, int G, int D, int Dv, int bs, float eps) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = qkv + t * qkv_stride;
  const long slot = slot_mapping[t];
  const long blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? (int)(slot % bs) : 0;
  for (int hv = wave; hv < H + G; hv += 4) {
    const T* x = row + (long)hv * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float a = (float)x[d];
      ss += a * a;
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)D + eps);
    if (hv < H) {
      for (int d = lane; d < D; d += 64) qn[(t * H + hv) * D + d] = (float)x[d] * r;
    } else if (slot >= 0) {
      const int c = hv - H;
      T* dst = k_cache + ((blk * G + c) * bs + off) * D;
      for (int d = lane; d < D; d += 64) dst[d] = (T)((float)x[d] * r);
    }
  }
  if (slot >= 0) {
    const T* v = row + (long)(H + G) * D;
    for (int e = threadIdx.x; e < G * Dv; e += 256) {
      const int c = e / Dv, d = e % Dv;
      v_cache[((blk * G + c) * bs + off) * Dv + d] = v[e];
    }
  }
}

VDA_EXPORT int vda_unit_rms_qk_cache(float* qn, const void* qkv, long qkv_stride, void* k_cache, void* v_cache,
                                     const long* slot_mapping, int T, int H, int G, int D, int Dv, int bs, float eps,
                                     int dtype, hipStream_t st) {
  if (T <= 0) return 0;
#define L(TT) hipLaunchKernelGGL((unit_rms_qk_cache_kernel<TT>), dim3(T), dim3(256), 0, st, qn, (const TT*)qkv, \
                                 qkv_stride, (TT*)k_cache, (TT*)v_cache, slot_mapping, H, G, D, Dv, bs, eps)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
  VDA_CHECK_LAUNCH();
  return 0;
}

// NACC: output values per thread (BQ * H * Dv <= 256 * NACC)
template <typename T, int NACC>
__global__ __launch_bounds__(256) void sigmoid_window_attention_kernel(
    T* __restrict__ out, const float* __restrict__ qn, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, long bt_stride, const int* __restrict__ seq_lens,
    const int* __restrict__ qsl, const float* __restrict__ talk, const float* __restrict__ pb, float scale,
    int window, int keep_first, int H, int G, int D, int Dv, int bs, int BQ, int BK) {
  extern __shared__ float lds[];
  const int Dq = (D + 3) / 4 * 4 + 4;           // padded row of q and k
  const int RS = BK + 1;                        // padded row of the score tiles
  float* qs = lds;                              // [BQ][H][Dq]
  float* ks = qs + BQ * H * Dq;                 // [BK][G][Dq]
  float* vs = ks + BK * G * Dq;                 // [BK][G][Dv]
  float* raw = vs + BK * G * Dv;                // [H][BQ][RS]
  float* wt = raw + H * BQ * RS;                // [H][BQ][RS]
  float* tk = wt + H * BQ * RS;                 // [H][H]
  float* pbs = tk + H * H;                      // [H]

  const int s = blockIdx.y, tid = threadIdx.x;
  const int sl = seq_lens[s];
  if (sl <= 0) return;
  const int t0 = qsl[s], L = qsl[s + 1] - t0;
  const int i0 = blockIdx.x * BQ;
  if (i0 >= L) return;
  const int nq = min(BQ, L - i0);
  const int p0 = sl - L + i0, p1 = p0 + nq;      // positions of the tile's queries: [p0, p1)
  const int rep = H / G;
  const int* bt = block_table + (long)s * bt_stride;

  for (int e = tid; e < H * H; e += 256) tk[e] = talk[e];
  for (int e = tid; e < H; e += 256) pbs[e] = pb[e];
  for (int e = tid; e < BQ * H * D; e += 256) {
    const int d = e % D, g = (e / D) % H, i = e / (D * H);
    qs[(i * H + g) * Dq + d] = i < nq ? qn[((long)(t0 + i0 + i) * H + g) * D + d] * scale : 0.f;
  }
  float acc[NACC];
#pragma unroll
  for (int n = 0; n < NACC; ++n) acc[n] = 0.f;

  // key ranges: the kept prefix [0, ka) and the window [lo, p1)
  const int lo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int ka = window > 0 ? min(min(keep_first, lo), p1) : 0;
  const int n_keep = (ka + BK - 1) / BK, n_win = (p1 - lo + BK - 1) / BK;
  for (int tile = 0; tile < n_keep + n_win; ++tile) {
    const int j0 = tile < n_keep ? tile * BK : lo + (tile - n_keep) * BK;
    const int jend = tile < n_keep ? ka : p1;
    const int nk = min(BK, jend - j0);
    __syncthreads();
    // K and V rows of the tile
    for (int e = tid; e < BK * G * D; e += 256) {
      const int d = e % D, c = (e / D) % G, jj = e / (D * G);
      float v = 0.f;
      if (jj < nk) {
        const int j = j0 + jj;
        v = (float)k_cache[(((long)bt[j / bs] * G + c) * bs + j % bs) * D + d];
      }
      ks[(jj * G + c) * Dq + d] = v;
    }
    for (int e = tid; e < BK * G * Dv; e += 256) {
      const int d = e % Dv, c = (e / Dv) % G, jj = e / (Dv * G);
      float v = 0.f;
      if (jj < nk) {
        const int j = j0 + jj;
        v = (float)v_cache[(((long)bt[j / bs] * G + c) * bs + j % bs) * Dv + d];
      }
      vs[(jj * G + c) * Dv + d] = v;
    }
    __syncthreads();
    // raw scores of every head
    for (int e = tid; e < H * BQ * BK; e += 256) {
      const int jj = e % BK, i = (e / BK) % BQ, g = e / (BK * BQ);
      const float* qp = qs + (i * H + g) * Dq;
      const float* kp = ks + (jj * G + g / rep) * Dq;
      float a = 0.f;
      for (int d = 0; d < D; ++d) a += qp[d] * kp[d];
      raw[(g * BQ + i) * RS + jj] = a;
    }
    __syncthreads();
    // mix over heads, weight function, visibility
    for (int e = tid; e < H * BQ * BK; e += 256) {
      const int jj = e % BK, i = (e / BK) % BQ, h = e / (BK * BQ);
      const int pi = p0 + i, j = j0 + jj;
      float w = 0.f;
      if (i < nq && jj < nk && j <= pi && (window <= 0 || pi - j < window || j < keep_first)) {
        float a = pbs[h];
        for (int g = 0; g < H; ++g) a += tk[h * H + g] * raw[(g * BQ + i) * RS + jj];
        w = 1.f / (1.f + expf(-a));
      }
      wt[(h * BQ + i) * RS + jj] = w;
    }
    __syncthreads();
    // weighted values
#pragma unroll
    for (int n = 0; n < NACC; ++n) {
      const int e = tid + n * 256;
      if (e < BQ * H * Dv) {
        const int d = e % Dv, h = (e / Dv) % H, i = e / (Dv * H);
        const float* wp = wt + (h * BQ + i) * RS;
        const float* vp = vs + (h / rep) * Dv + d;
        float a = acc[n];
        for (int jj = 0; jj < nk; ++jj) a += wp[jj] * vp[jj * G * Dv];
        acc[n] = a;
      }
    }
  }
#pragma unroll
  for (int n = 0; n < NACC; ++n) {
    const int e = tid + n * 256;
    if (e < BQ * H * Dv) {
      const int hd = e % (Dv * H), i = e / (Dv * H);
      if (i < nq) out[(long)(t0 + i0 + i) * H * Dv + hd] = (T)acc[n];
    }
  }
}

VDA_EXPORT int vda_sigmoid_window_attention(void* out, const float* qn, const void* k_cache, const void* v_cache,
                                            const int* block_table, long bt_stride, const int* seq_lens,
                                            const int* qsl, const float* talk, const float* pb, float scale,
                                            int window, int keep_first, int S, int H, int G, int D, int Dv, int bs,
                                            int max_q, int dtype, hipStream_t st) {
  if (S <= 0 || max_q <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G) return -1;
  // query tile: as many tokens as the per-thread accumulators (64) and 96 KiB of LDS allow
  const int Dq = (D + 3) / 4 * 4 + 4;
  int BQ = 16, BK = 32;
  auto lds_of = [&](int bq, int bk) {
    return ((size_t)bq * H * Dq + (size_t)bk * G * (Dq + Dv) + 2 * (size_t)H * bq * (bk + 1) + (size_t)H * H + H) * 4;
  };
  while (BQ > 1 && (BQ > max_q * 2 - 1 || (size_t)BQ * H * Dv > 256 * 64 || lds_of(BQ, 16) > 96 * 1024)) BQ >>= 1;
  if (BQ > 1 && BQ / 2 >= max_q) BQ >>= 1;
  if ((size_t)BQ * H * Dv > 256 * 64) return -2;
  if (lds_of(BQ, BK) > 96 * 1024) BK = 16;
  const size_t lds = lds_of(BQ, BK);
  if (lds > 96 * 1024) return -2;
  const int per = (BQ * H * Dv + 255) / 256;
  const int NACC = per <= 8 ? 8 : per <= 16 ? 16 : per <= 32 ? 32 : 64;
  dim3 grid((max_q + BQ - 1) / BQ, S), block(256);
#define L2(TT, NA)                                                                                                  \
  do {                                                                                                              \
    if (lds > 48 * 1024) {                                                                                          \
      hipError_t e = hipFuncSetAttribute((const void*)sigmoid_window_attention_kernel<TT, NA>,                     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                     \
      if (e != hipSuccess) return (int)e;                                                                           \
    }                                                                                                               \
    hipLaunchKernelGGL((sigmoid_window_attention_kernel<TT, NA>), grid, block, lds, st, (TT*)out, qn,               \
                       (const TT*)k_cache, (const TT*)v_cache, block_table, bt_stride, seq_lens, qsl, talk, pb,     \
                       scale, window, keep_first, H, G, D, Dv, bs, BQ, BK);                                         \
  } while (0)
#define L(TT)                                                                                                       \
  do {                                                                                                              \
    if (NACC == 8) L2(TT, 8); else if (NACC == 16) L2(TT, 16); else if (NACC == 32) L2(TT, 32); else L2(TT, 64);    \
  } while (0)
  if (dtype == VDA_BF16) L(bf16_t);
  else if (dtype == VDA_F16) L(f16_t);
  else if (dtype == VDA_F32) L(float);
  else return -3;
#undef L
#undef L2
  VDA_CHECK_LAUNCH();
  return 0;
}
