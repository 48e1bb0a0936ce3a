// Sigmoid attention with mixed head scores ("talking heads" before the weight function), over a sliding window
// plus the first tokens of the sequence, on the paged cache.  No softmax: nothing is normalised over keys.
//
//   raw[g](i, j)  = scale * qn[i, g] . kn[j, kv(g)]          qn, kn: per-head RMS-normalised, no learned weight
//   s[h](i, j)    = sum_g talk[h, g] raw[g](i, j) + pb[h]
//   out[i, h]     = sum over visible j of sigmoid(s[h](i, j)) * v[j, kv(h)]
//   visible: j <= i and (i - j < window or j < keep_first); window == 0: every j <= i
//
// Cache layout (the framework's): k_cache [blocks, G, block_size, D], v_cache [blocks, G, Dv, block_size]; key and
// value widths may differ.
//
//   vda_unit_rms_qk_cache         q -> qn ([T, H, D], the activation type); kn and v -> cache at slot_mapping
//   vda_sigmoid_window_attention  one workgroup per (sequence, tile of query tokens); scores, mixing and the weight
//                                 function in fp32; keys outside the window and the kept prefix are never loaded.
//                                 Prompts, portions of prompts and single decoded tokens are one code path.
//     * fp32 activations, odd sizes, single tokens: plain fp32 arithmetic through LDS tiles
//     * 16-bit activations with 16 query tokens per tile: MFMA for q.k and weights.v, the mixing on the vector
//       units from registers (see sigmoid_attention_mfma_kernel)
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void unit_rms_qk_cache_kernel(
    T* __restrict__ qn, const T* __restrict__ qkv, long qkv_stride, T* __restrict__ k_cache,
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
      for (int d = lane; d < D; d += 64) qn[(t * H + hv) * D + d] = (T)((float)x[d] * r);
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
      v_cache[((blk * G + c) * Dv + d) * bs + off] = v[e];
    }
  }
}

VDA_EXPORT int vda_unit_rms_qk_cache(void* qn, const void* qkv, long qkv_stride, void* k_cache, void* v_cache,
                                     const long* slot_mapping, int T, int H, int G, int D, int Dv, int bs, float eps,
                                     int dtype, hipStream_t st) {
  if (T <= 0) return 0;
#define L(TT) hipLaunchKernelGGL((unit_rms_qk_cache_kernel<TT>), dim3(T), dim3(256), 0, st, (TT*)qn, (const TT*)qkv, \
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
    T* __restrict__ out, const T* __restrict__ qn, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
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
    qs[(i * H + g) * Dq + d] = i < nq ? (float)qn[((long)(t0 + i0 + i) * H + g) * D + d] * scale : 0.f;
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
        v = (float)v_cache[(((long)bt[j / bs] * G + c) * Dv + d) * bs + j % bs];
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

// ---- MFMA form (16-bit activations) ---------------------------------------------------------------------
// One workgroup = one sequence x 16 query tokens x ALL heads; a step covers 128 keys, 32 per wave.
//   1. every wave: S^T = K . Q^T for its 32 keys and every head (A = key rows straight from the cache, B = the
//      queries from LDS), so a lane ends up with the scores of ONE query (column r = lane & 15) for 8 consecutive
//      keys (8 (lane >> 4) ..) of every head, in registers;
//   2. the same wave mixes them over heads (fp32, weights from LDS), adds the bias, applies the sigmoid and the
//      visibility, and leaves the 8 weights of every head as one 16-byte row in LDS -- already in the layout of an
//      MFMA B operand (the mixing weights sit in LDS too: one broadcast read per four heads);
//   3. after a barrier the waves change roles: wave w owns heads [w H/4, (w+1) H/4) and accumulates
//      O^T += V^T . P^T over the four 32-key parts (A = value rows with 8 contiguous keys, which is what the
//      cache's V layout stores).
// MAXH: heads rounded up to 8 or 16; KS: 32-wide steps over the key width; NT: 16-wide tiles of the value width.
template <typename T, int MAXH, int KS, int NT>
__global__ __launch_bounds__(256) void sigmoid_attention_mfma_kernel(
    T* __restrict__ out, const T* __restrict__ qn, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, long bt_stride, const int* __restrict__ seq_lens,
    const int* __restrict__ qsl, const float* __restrict__ talk, const float* __restrict__ pb, float scale,
    int window, int keep_first, int H, int G, int D, int Dv, int bs, float* __restrict__ part, long part_stride) {
  using V8 = typename Vec<T>::v8;
  constexpr int HPW = MAXH / 4;                 // heads a wave accumulates
  extern __shared__ __align__(16) unsigned char smem[];
  V8* pl = reinterpret_cast<V8*>(smem);         // [MAXH][4][64] weights, 16 bytes each
  float* tk = reinterpret_cast<float*>(smem + (size_t)MAXH * 4 * 64 * 16);    // [MAXH][MAXH] mixing weights x scale
  float* pbs = tk + MAXH * MAXH;                                              // [MAXH]

  const int s = blockIdx.y, tid = threadIdx.x;
  const int sl = seq_lens[s];
  if (sl <= 0) return;
  const int t0 = qsl[s], L = qsl[s + 1] - t0;
  const int i0 = blockIdx.x * 16;
  if (i0 >= L) return;
  const int nq = min(16, L - i0);
  const int p0 = sl - L + i0, p1 = p0 + nq;
  const int rep = H / G;
  const int* bt = block_table + (long)s * bt_stride;
  const int nblk = (sl + bs - 1) / bs;
  const int lane = tid & 63, wave = tid >> 6, r = lane & 15, g4 = lane >> 4;

  for (int e = tid; e < MAXH * MAXH; e += 256) {
    const int hh = e / MAXH, gg = e % MAXH;
    tk[e] = (hh < H && gg < H) ? talk[hh * H + gg] * scale : 0.f;
  }
  for (int e = tid; e < MAXH; e += 256) pbs[e] = e < H ? pb[e] : 0.f;
  __syncthreads();
  // this lane's query row (columns beyond the tile repeat the last one; they are masked and never stored)
  const T* qrow = qn + (long)(t0 + i0 + min(r, nq - 1)) * H * D;
  V8 zero8;
#pragma unroll
  for (int j = 0; j < 8; ++j) zero8[j] = (T)0.f;
  f32x4 acc[HPW][NT];
#pragma unroll
  for (int a = 0; a < HPW; ++a)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[a][n] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int lo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int ka = window > 0 ? min(min(keep_first, lo), p1) : 0;
  const int lo_al = lo & ~31;
  const int n_keep = (ka + 127) / 128, n_win = (p1 - lo_al + 127) / 128;
  const int krow0 = 8 * (r >> 2) + (r & 3);
  const int pi = p0 + r;                        // position of this lane's query column
  // few query tiles (decoding): the key steps are dealt to gridDim.z workgroups, whose partial sums -- nothing is
  // normalised over keys, so they simply add -- go to `part` and are summed in a fixed order afterwards
  for (int step = blockIdx.z; step < n_keep + n_win; step += gridDim.z) {
    const bool keep = step < n_keep;
    const int kb = keep ? step * 128 : lo_al + (step - n_keep) * 128;
    const int jlo = keep ? 0 : lo, jhi = keep ? ka : p1;        // keys of this range that count
    const int tb = kb + 32 * wave;
    // ---- scores of every head for this wave's 32 keys ----------------------------------------------------------
    float raw[MAXH][8];
    if (tb < jhi && tb + 32 > jlo) {
      V8 kf[2][KS];
#pragma unroll
      for (int h = 0; h < MAXH; ++h) {
        if (h < H) {
          if (h % rep == 0) {
            const int c = h / rep;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
              const int tok = tb + krow0 + 4 * u;
              const long blk = bt[min(tok / bs, nblk - 1)];
              const T* kp = k_cache + ((blk * G + c) * bs + tok % bs) * (long)D;
#pragma unroll
              for (int ks = 0; ks < KS; ++ks) {
                const int d0 = (ks * 4 + g4) * 8;
                kf[u][ks] = ld16<V8>(kp + (d0 < D ? d0 : 0));
              }
            }
          }
          f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const int d0 = (ks * 4 + g4) * 8;
            const V8 qf = d0 < D ? ld16<V8>(qrow + (long)h * D + d0) : zero8;
            s0 = mfma16(kf[0][ks], qf, s0);
            s1 = mfma16(kf[1][ks], qf, s1);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            raw[h][j] = s0[j];
            raw[h][4 + j] = s1[j];
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) raw[h][j] = 0.f;
        }
      }
      // ---- mix over heads, weight function, visibility -> LDS -----------------------------------------------------
      bool vis[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = tb + 8 * g4 + j;
        vis[j] = r < nq && key >= jlo && key < jhi && key <= pi &&
                 (window <= 0 || pi - key < window || key < keep_first);
      }
#pragma unroll
      for (int h = 0; h < MAXH; ++h) {
        if (h < H) {
          float m[8];
          const float bias = pbs[h];
#pragma unroll
          for (int j = 0; j < 8; ++j) m[j] = bias;
#pragma unroll
          for (int g4i = 0; g4i < MAXH / 4; ++g4i) {          // one broadcast 16-byte LDS read per four heads
            const f32x4 w4 = *reinterpret_cast<const f32x4*>(tk + h * MAXH + 4 * g4i);
#pragma unroll
            for (int gg = 0; gg < 4; ++gg)
#pragma unroll
              for (int j = 0; j < 8; ++j) m[j] += w4[gg] * raw[4 * g4i + gg][j];
          }
          V8 pv;
#pragma unroll
          for (int j = 0; j < 8; ++j) pv[j] = (T)(vis[j] ? 1.f / (1.f + __expf(-m[j])) : 0.f);
          pl[(h * 4 + wave) * 64 + lane] = pv;
        }
      }
    } else {
      V8 z;
#pragma unroll
      for (int j = 0; j < 8; ++j) z[j] = (T)0.f;
#pragma unroll
      for (int h = 0; h < MAXH; ++h)
        if (h < H) pl[(h * 4 + wave) * 64 + lane] = z;
    }
    __syncthreads();
    // ---- weighted values: this wave's heads over the step's four key parts ------------------------------------
#pragma unroll
    for (int w2 = 0; w2 < 4; ++w2) {
      const int tb2 = kb + 32 * w2;
      if (tb2 < jhi && tb2 + 32 > jlo) {
        const int tok = tb2 + 8 * g4;
        const long blk = bt[min(tok / bs, nblk - 1)];
        int c_prev = -1;
        V8 vf[NT];
#pragma unroll
        for (int a = 0; a < HPW; ++a) {
          const int h = wave * HPW + a;
          if (h < H) {
            const int c = h / rep;
            if (c != c_prev) {
              c_prev = c;
#pragma unroll
              for (int n = 0; n < NT; ++n) {
                const int d = min(n * 16 + r, Dv - 1);
                vf[n] = ld16<V8>(v_cache + ((blk * G + c) * (long)Dv + d) * bs + tok % bs);
              }
            }
            const V8 pv = pl[(h * 4 + w2) * 64 + lane];
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[a][n] = mfma16(vf[n], pv, acc[a][n]);
          }
        }
      }
    }
    __syncthreads();
  }
  // O^T tiles: the lane holds value columns n*16 + 4 g4 + j of query r
  if (r < nq) {
#pragma unroll
    for (int a = 0; a < HPW; ++a) {
      const int h = wave * HPW + a;
      if (h < H) {
        const long at = (long)(t0 + i0 + r) * H * Dv + (long)h * Dv;
#pragma unroll
        for (int n = 0; n < NT; ++n)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int d = n * 16 + 4 * g4 + j;
            if (d < Dv) {
              if (part) part[blockIdx.z * part_stride + at + d] = acc[a][n][j];
              else out[at + d] = (T)acc[a][n][j];
            }
          }
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void sum_parts_kernel(T* __restrict__ out, const float* __restrict__ part,
                                                        long n, long part_stride, int parts) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float a = 0.f;
  for (int z = 0; z < parts; ++z) a += part[z * part_stride + i];
  out[i] = (T)a;
}

template <typename T>
static int launch_sigmoid_mfma(dim3 grid, hipStream_t st, void* out, const void* qn, const void* k_cache,
                               const void* v_cache, const int* block_table, long bt_stride, const int* seq_lens,
                               const int* qsl, const float* talk, const float* pb, float scale, int window,
                               int keep_first, int H, int G, int D, int Dv, int bs, float* part, long part_stride) {
  const int MAXH = H <= 8 ? 8 : 16, KS = D <= 64 ? 2 : 4, NT = Dv <= 64 ? 4 : 8;
  const size_t lds = (size_t)MAXH * 4 * 64 * 16 + ((size_t)MAXH * MAXH + MAXH) * 4;
#define LM(MH, KK, NN)                                                                                              \
  do {                                                                                                              \
    if (lds > 48 * 1024) {                                                                                          \
      hipError_t e = hipFuncSetAttribute((const void*)sigmoid_attention_mfma_kernel<T, MH, KK, NN>,                \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                     \
      if (e != hipSuccess) { (void)hipGetLastError(); return -1000 - (int)e; }                                      \
    }                                                                                                               \
    hipLaunchKernelGGL((sigmoid_attention_mfma_kernel<T, MH, KK, NN>), grid, dim3(256), lds, st, (T*)out,           \
                       (const T*)qn,                                                                                \
                       (const T*)k_cache, (const T*)v_cache, block_table, bt_stride, seq_lens, qsl, talk, pb,       \
                       scale, window, keep_first, H, G, D, Dv, bs, part, part_stride);                              \
  } while (0)
#define LK(MH, KK) do { if (NT == 4) LM(MH, KK, 4); else LM(MH, KK, 8); } while (0)
#define LH(MH) do { if (KS == 2) LK(MH, 2); else LK(MH, 4); } while (0)
  if (MAXH == 8) LH(8); else LH(16);
#undef LH
#undef LK
#undef LM
  if (part) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL((sum_parts_kernel<T>), dim3((unsigned)((part_stride + 255) / 256)), dim3(256), 0, st, (T*)out,
                       part, part_stride, part_stride, (int)grid.z);
  }
  return 0;
}

// 1: the MFMA form takes this problem (16-bit, sizes it is built for, block sizes that keep 8 keys in one page)
VDA_EXPORT int vda_sigmoid_attention_mfma_ok(int H, int G, int D, int Dv, int bs, int dtype) {
  return (dtype == VDA_BF16 || dtype == VDA_F16) && H >= 1 && H <= 16 && G >= 1 && H % G == 0 && D % 8 == 0 &&
         D <= 128 && Dv % 8 == 0 && Dv <= 128 && bs % 8 == 0;
}

VDA_EXPORT int vda_sigmoid_window_attention(void* out, const void* qn, const void* k_cache, const void* v_cache,
                                            const int* block_table, long bt_stride, const int* seq_lens,
                                            const int* qsl, const float* talk, const float* pb, float scale,
                                            int window, int keep_first, int S, int H, int G, int D, int Dv, int bs,
                                            int max_q, int dtype, int form, float* part, long part_stride,
                                            int parts, hipStream_t st) {
  if (S <= 0 || max_q <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G) return -1;
  if (form == 1) {              // MFMA form
    if (!vda_sigmoid_attention_mfma_ok(H, G, D, Dv, bs, dtype)) return -2;
    // parts > 1: `part` holds parts x part_stride zeroed floats (part_stride = tokens * H * Dv)
    dim3 grid((max_q + 15) / 16, S, part && parts > 1 ? parts : 1);
    float* pp = grid.z > 1 ? part : nullptr;
    int rc = dtype == VDA_BF16
                 ? launch_sigmoid_mfma<bf16_t>(grid, st, out, qn, k_cache, v_cache, block_table, bt_stride, seq_lens,
                                               qsl, talk, pb, scale, window, keep_first, H, G, D, Dv, bs, pp,
                                               part_stride)
                 : launch_sigmoid_mfma<f16_t>(grid, st, out, qn, k_cache, v_cache, block_table, bt_stride, seq_lens,
                                              qsl, talk, pb, scale, window, keep_first, H, G, D, Dv, bs, pp,
                                              part_stride);
    if (rc) return rc;
    VDA_CHECK_LAUNCH();
    return 0;
  }
  // tile sizes: the largest query tile (then key tile) whose accumulators fit 64 registers per thread and whose
  // tiles fit 96 KiB of LDS; single decoded tokens take a one-token tile
  const int Dq = (D + 3) / 4 * 4 + 4;
  auto lds_of = [&](int bq, int bk) {
    return ((size_t)bq * H * Dq + (size_t)bk * G * (Dq + Dv) + 2 * (size_t)H * bq * (bk + 1) + (size_t)H * H + H) * 4;
  };
  int BQ = 0, BK = 0;
  for (int bq = 16; bq >= 1 && !BQ; bq >>= 1) {
    if (bq > 1 && bq / 2 >= max_q) continue;
    if ((size_t)bq * H * Dv > 256 * 64) continue;
    for (int bk = 32; bk >= 1; bk >>= 1)
      if (lds_of(bq, bk) <= 96 * 1024) { BQ = bq; BK = bk; break; }
  }
  if (!BQ) return -2;
  const size_t lds = lds_of(BQ, BK);
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
    hipLaunchKernelGGL((sigmoid_window_attention_kernel<TT, NA>), grid, block, lds, st, (TT*)out, (const TT*)qn,    \
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
