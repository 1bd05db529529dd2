// Sequence-mixing kernels of the hybrid decoders (gfx950, wave64).
//
//   latent attention   one cached row per token [latent c (r) | rotated key
//                      (dr)], shared by all heads; scores, softmax and the
//                      weighted sum of latents in f32; ragged batches (every
//                      token carries its sequence and position), paged rows
//   mLSTM scan         matrix memory S [d, dv] + normaliser n [d] + running
//                      maximum m per (sequence, head), f32, carried in state
//                      slots between steps; token-sequential inside a step
//   element-wise       hashed-bigram embedding, scaled LayerNorm-on-output
//                      residual add (f32 stream), latent RMSNorm + rotary +
//                      cache append, rotary on query rows, per-head RMSNorm *
//                      weight * sigmoid gate, tanh-GELU GLU
//
// Activations are bf16 or f32 (template E); accumulation is always f32.
#include "seqmix.h"

#include <math.h>

namespace illm {
namespace sm {
namespace {

template <typename E> __device__ __forceinline__ float ldf(const E* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<__bf16>(const __bf16* p) { return (float)*p; }
template <typename E> __device__ __forceinline__ void stf(E* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<__bf16>(__bf16* p, float v) { *p = (__bf16)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// LDS written by some lanes of a wave becomes visible to its other lanes
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
// sum over a block of up to 1024 threads; red: >= 16 floats of LDS
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nw; i++) s += red[i];
  return s;
}

// ------------------------------------------------------------------ embedding
template <typename E>
__global__ void __launch_bounds__(256) embed_bigram_k(const int64_t* __restrict__ ids, const int64_t* __restrict__ prev,
                                                     const E* __restrict__ embed, const E* __restrict__ bigram,
                                                     float* __restrict__ out, int W, int64_t vocab, int64_t buckets,
                                                     int64_t mp, int64_t mc) {
  const int t = blockIdx.x;
  const int64_t id = ids[t], p = prev[t];
  float* o = out + (int64_t)t * W;
  if (id < 0 || id >= vocab) {                    // bad id: a zero row, never an out-of-bounds read
    for (int c = threadIdx.x; c < W; c += blockDim.x) o[c] = 0.f;
    return;
  }
  const int64_t row = p < 0 ? buckets : ((p * mp + id * mc) % buckets);
  const E* e = embed + id * W;
  const E* b = bigram + row * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) o[c] = ldf(e + c) + ldf(b + c);
}

// ------------------------------------------------------------------ norms
template <typename E>
__global__ void __launch_bounds__(256) add_sln_k(float* __restrict__ x, const E* __restrict__ y, const E* __restrict__ w,
                                                E* __restrict__ xa, int W, float eps, float mult) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const E* yr = y + t * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) s += ldf(yr + c);
  const float mean = block_sum(s, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = ldf(yr + c) - mean;
    q += d * d;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
  float* xr = x + t * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = xr[c] + mult * ((ldf(yr + c) - mean) * rs * ldf(w + c));
    xr[c] = v;
    if (xa) stf(xa + t * W + c, v);
  }
}

template <typename E>
__global__ void __launch_bounds__(256) layer_norm_k(const float* __restrict__ x, const E* __restrict__ w,
                                                   E* __restrict__ out, int W, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float* xr = x + t * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) s += xr[c];
  const float mean = block_sum(s, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = xr[c] - mean;
    q += d * d;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(out + t * W + c, (xr[c] - mean) * rs * ldf(w + c));
}

// ------------------------------------------------------------------ rotary
template <typename E>
__global__ void __launch_bounds__(256) rope_rows_k(E* __restrict__ q, int H, int Dh, int offset,
                                                  const float* __restrict__ table, int max_pos, int dims,
                                                  const int64_t* __restrict__ pos) {
  const int64_t t = blockIdx.x;
  const int64_t p = pos[t];
  if (p < 0 || p >= max_pos) return;
  const int half = dims >> 1;
  const float* cs = table + p * dims;             // [half][2]
  for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
    const int h = i / half, k = i - h * half;
    E* a = q + (t * H + h) * Dh + offset + 2 * k;
    const float u = ldf(a), v = ldf(a + 1), c = cs[2 * k], s = cs[2 * k + 1];
    stf(a, u * c - v * s);
    stf(a + 1, v * c + u * s);
  }
}

template <typename E>
__global__ void __launch_bounds__(128) latent_kv_store_k(const E* __restrict__ dkv, int64_t ld, const E* __restrict__ nw,
                                                        float eps, int r, int dr, const float* __restrict__ table,
                                                        int max_pos, int dims, const int64_t* __restrict__ pos,
                                                        const int64_t* __restrict__ slots, E* __restrict__ rows,
                                                        int64_t num_rows) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int64_t slot = slots[t], p = pos[t];
  const E* in = dkv + t * ld;
  float q = 0.f;
  for (int c = threadIdx.x; c < r; c += blockDim.x) {
    const float v = ldf(in + c);
    q += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)r + eps);
  if (slot < 0 || slot >= num_rows || p < 0 || p >= max_pos) return;      // padded row
  E* out = rows + slot * (int64_t)(r + dr);
  for (int c = threadIdx.x; c < r; c += blockDim.x) stf(out + c, ldf(in + c) * rs * ldf(nw + c));
  const float* cs = table + p * dims;
  const int half = dims >> 1;
  for (int k = threadIdx.x; k < half; k += blockDim.x) {
    const float u = ldf(in + r + 2 * k), v = ldf(in + r + 2 * k + 1), c = cs[2 * k], s = cs[2 * k + 1];
    stf(out + r + 2 * k, u * c - v * s);
    stf(out + r + 2 * k + 1, v * c + u * s);
  }
  for (int c = dims + threadIdx.x; c < dr; c += blockDim.x) stf(out + r + c, ldf(in + r + c));
}

// ------------------------------------------------------------------ latent attention
// One workgroup: one query token x up to HB heads.  Its NW waves walk the
// token's key tiles (KT keys each, tile i -> keys [i KT, (i + 1) KT), always
// inside one cache page) round-robin; a wave stages a tile in LDS, lane j
// scores key j against every head (f32), the wave does the online-softmax
// update per head, and every lane accumulates its latent columns.  The waves'
// partial (max, sum, out) are merged through LDS at the end.
constexpr int HB = 8;

template <typename E, int RC>
__global__ void __launch_bounds__(256) latent_attn_k(const E* __restrict__ q_lat, const E* __restrict__ q_rot,
                                                    int64_t qr_st, int64_t qr_sh, const E* __restrict__ rows, int bs,
                                                    const int32_t* __restrict__ bt, int bt_w,
                                                    const int32_t* __restrict__ seq_of, const int64_t* __restrict__ pos,
                                                    float scale, const E* __restrict__ gate, int64_t g_st,
                                                    E* __restrict__ out, int H, int r, int dr, int KT, int DP) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int D = r + dr;
  const int t = blockIdx.x, h0 = blockIdx.y * HB;
  const int nh = min(HB, H - h0);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  float* qs = (float*)smem;                                        // [HB][D]
  const size_t wave_bytes = ((size_t)KT * DP * sizeof(E) + (size_t)HB * KT * sizeof(float) + 15) & ~(size_t)15;
  unsigned char* wbase = smem + (((size_t)HB * D * sizeof(float) + 15) & ~(size_t)15) + wv * wave_bytes;
  E* kt = (E*)wbase;                                               // [KT][DP]
  float* pb = (float*)(wbase + (size_t)KT * DP * sizeof(E));       // [HB][KT]
  for (int i = threadIdx.x; i < HB * D; i += blockDim.x) {
    const int h = i / D, c = i - h * D;
    float v = 0.f;
    if (h < nh) v = c < r ? ldf(q_lat + ((int64_t)t * H + h0 + h) * r + c)
                          : ldf(q_rot + (int64_t)t * qr_st + (int64_t)(h0 + h) * qr_sh + (c - r));
    qs[i] = v;
  }
  __syncthreads();
  const int64_t p = pos[t];
  const int32_t* tab = bt + (int64_t)seq_of[t] * bt_w;
  const int ntiles = (int)(p / KT) + 1;
  float m[HB], l[HB], o[HB][RC];
#pragma unroll
  for (int h = 0; h < HB; h++) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int c = 0; c < RC; c++) o[h][c] = 0.f;
  }
  for (int ti = wv; ti < ntiles; ti += NW) {
    const int64_t k0 = (int64_t)ti * KT;
    const int nvalid = (int)min((int64_t)KT, p - k0 + 1);
    const int64_t row0 = (int64_t)tab[k0 / bs] * bs + (k0 % bs);
    const E* src = rows + row0 * D;
    for (int i = lane; i < nvalid * D; i += 64) {
      const int j = i / D, c = i - j * D;
      kt[j * DP + c] = src[i];
    }
    wave_sync();                                                   // the tile is in LDS
    float s[HB];
#pragma unroll
    for (int h = 0; h < HB; h++) s[h] = 0.f;
    const bool valid = lane < nvalid;
    if (valid) {
      const E* kr = kt + lane * DP;
      for (int c = 0; c < D; c++) {
        const float kv = ldf(kr + c);
#pragma unroll
        for (int h = 0; h < HB; h++) s[h] = fmaf(qs[h * D + c], kv, s[h]);
      }
    }
#pragma unroll
    for (int h = 0; h < HB; h++) {
      const float sv = valid ? s[h] * scale : -INFINITY;
      const float mn = fmaxf(m[h], wave_max(sv));
      const float alpha = m[h] == -INFINITY ? 0.f : expf(m[h] - mn);
      const float pv = valid ? expf(sv - mn) : 0.f;
      l[h] = l[h] * alpha + wave_sum(pv);
      m[h] = mn;
#pragma unroll
      for (int c = 0; c < RC; c++) o[h][c] *= alpha;
      if (lane < KT) pb[h * KT + lane] = pv;
    }
    wave_sync();
    for (int j = 0; j < nvalid; j++) {
      float kv[RC];
#pragma unroll
      for (int c = 0; c < RC; c++) {
        const int col = lane + 64 * c;
        kv[c] = col < r ? ldf(kt + j * DP + col) : 0.f;
      }
#pragma unroll
      for (int h = 0; h < HB; h++) {
        const float pv = pb[h * KT + j];
#pragma unroll
        for (int c = 0; c < RC; c++) o[h][c] = fmaf(pv, kv[c], o[h][c]);
      }
    }
    wave_sync();
  }
  // merge the waves: every wave leaves (m, l, o) in its own LDS region
  float* mg = (float*)wbase;                                       // [HB][r + 2]
#pragma unroll
  for (int h = 0; h < HB; h++) {
#pragma unroll
    for (int c = 0; c < RC; c++) {
      const int col = lane + 64 * c;
      if (col < r) mg[h * (r + 2) + col] = o[h][c];
    }
    if (lane == 0) {
      mg[h * (r + 2) + r] = m[h];
      mg[h * (r + 2) + r + 1] = l[h];
    }
  }
  __syncthreads();
  unsigned char* w0 = smem + (((size_t)HB * D * sizeof(float) + 15) & ~(size_t)15);
  for (int i = threadIdx.x; i < nh * r; i += blockDim.x) {
    const int h = i / r, c = i - h * r;
    float M = -INFINITY;
    for (int w = 0; w < NW; w++) M = fmaxf(M, ((const float*)(w0 + w * wave_bytes))[h * (r + 2) + r]);
    float L = 0.f, O = 0.f;
    for (int w = 0; w < NW; w++) {
      const float* g = (const float*)(w0 + w * wave_bytes) + h * (r + 2);
      const float mw = g[r];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      L += g[r + 1] * f;
      O += g[c] * f;
    }
    float v = O / L;
    if (gate) v *= 1.0f / (1.0f + expf(-ldf(gate + (int64_t)t * g_st + h0 + h)));
    stf(out + ((int64_t)t * H + h0 + h) * r + c, v);
  }
}

// ------------------------------------------------------------------ mLSTM
// One wave: 64 value columns of one (sequence, head).  S [d][64] lives in LDS
// column-per-lane; n [d] is kept redundantly by every column block.
template <typename E>
__global__ void __launch_bounds__(64) mlstm_scan_k(const E* __restrict__ q, int64_t q_ld, const E* __restrict__ k,
                                                  int64_t k_ld, const E* __restrict__ v, int64_t v_ld,
                                                  const E* __restrict__ ipre, int64_t i_ld, const E* __restrict__ fpre,
                                                  int64_t f_ld, const float* __restrict__ ib, const float* __restrict__ fb,
                                                  float cap, float* __restrict__ Sg, float* __restrict__ ng,
                                                  float* __restrict__ mgl, const int32_t* __restrict__ cu,
                                                  const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
                                                  float* __restrict__ out, int H, int d, int dv) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* S = (float*)smem;                 // [d][64]
  float* nb = S + (size_t)d * 64;          // [d]
  float* qb = nb + d;                      // [d]
  float* kb = qb + d;                      // [d]
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int j = blockIdx.z * 64 + lane;
  const bool jv = j < dv;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t0 >= t1) return;
  const int64_t slot = slots[b];
  const bool fresh = pos[t0] == 0;
  float* Ss = Sg + ((slot * H + h) * d) * (int64_t)dv;
  float* ns = ng + (slot * H + h) * (int64_t)d;
  float m = fresh ? 0.f : mgl[slot * H + h];
  for (int dd = 0; dd < d; dd++) S[dd * 64 + lane] = (fresh || !jv) ? 0.f : Ss[(int64_t)dd * dv + j];
  for (int dd = lane; dd < d; dd += 64) nb[dd] = fresh ? 0.f : ns[dd];
  const float qscale = 1.0f / sqrtf((float)d);
  for (int t = t0; t < t1; t++) {
    __syncthreads();
    for (int dd = lane; dd < d; dd += 64) {
      qb[dd] = ldf(q + (int64_t)t * q_ld + h * d + dd) * qscale;
      kb[dd] = ldf(k + (int64_t)t * k_ld + h * d + dd);
    }
    const float iz = (ldf(ipre + (int64_t)t * i_ld + h) + ib[h]) / cap;
    const float fz = cap * tanhf((ldf(fpre + (int64_t)t * f_ld + h) + fb[h]) / cap);
    const float ig = cap * tanhf(iz);
    const float fg = fminf(fz, 0.f) - log1pf(expf(-fabsf(fz)));    // logsigmoid
    const float mn = fmaxf(fg + m, ig);
    const float a = expf(fg + m - mn), bb = expf(ig - mn);
    m = mn;
    const float vj = jv ? ldf(v + (int64_t)t * v_ld + h * dv + j) : 0.f;
    __syncthreads();
    float acc = 0.f;
    for (int dd = 0; dd < d; dd++) {
      const float s = a * S[dd * 64 + lane] + (bb * kb[dd]) * vj;
      S[dd * 64 + lane] = s;
      acc = fmaf(s, qb[dd], acc);
    }
    float part = 0.f;
    for (int dd = lane; dd < d; dd += 64) {
      const float nn = a * nb[dd] + bb * kb[dd];
      nb[dd] = nn;
      part = fmaf(nn, qb[dd], part);
    }
    const float nq = wave_sum(part);
    const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
    if (jv) out[((int64_t)t * H + h) * dv + j] = acc / den;
  }
  __syncthreads();
  if (jv)
    for (int dd = 0; dd < d; dd++) Ss[(int64_t)dd * dv + j] = S[dd * 64 + lane];
  if (blockIdx.z == 0) {
    for (int dd = lane; dd < d; dd += 64) ns[dd] = nb[dd];
    if (lane == 0) mgl[slot * H + h] = m;
  }
}

template <typename E>
__global__ void __launch_bounds__(64) head_rms_gate_k(const float* __restrict__ hh, const E* __restrict__ nw,
                                                     const E* __restrict__ gate, int64_t g_ld, E* __restrict__ out,
                                                     int H, int dv, float eps) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* in = hh + (t * H + h) * dv;
  float q = 0.f;
  for (int c = threadIdx.x; c < dv; c += 64) q += in[c] * in[c];
  const float rs = 1.0f / sqrtf(wave_sum(q) / (float)dv + eps);
  for (int c = threadIdx.x; c < dv; c += 64) {
    const float g = 1.0f / (1.0f + expf(-ldf(gate + t * g_ld + h * dv + c)));
    stf(out + (t * H + h) * dv + c, in[c] * rs * ldf(nw + h * dv + c) * g);
  }
}

template <typename E>
__global__ void __launch_bounds__(256) glu_gelu_k(const E* __restrict__ gu, E* __restrict__ out, int64_t T, int64_t I) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * I) return;
  const int64_t t = i / I, c = i - t * I;
  const float g = ldf(gu + t * 2 * I + c), u = ldf(gu + t * 2 * I + I + c);
  const float a = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  stf(out + i, a * u);
}

}  // namespace

#define SM_DISPATCH(bf16, ...)                 \
  if (bf16) {                                  \
    typedef __bf16 E;                          \
    __VA_ARGS__;                               \
  } else {                                     \
    typedef float E;                           \
    __VA_ARGS__;                               \
  }

void embed_bigram(bool bf16, const int64_t* ids, const int64_t* prev, const void* embed, const void* bigram, float* out,
                  int T, int W, int64_t vocab, int64_t buckets, int64_t mul_prev, int64_t mul_cur, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(embed_bigram_k<E>, dim3(T), dim3(256), 0, st, ids, prev, (const E*)embed,
                                       (const E*)bigram, out, W, vocab, buckets, mul_prev, mul_cur));
}

void add_scaled_layer_norm(bool bf16, float* x, const void* y, const void* w, void* xa, int T, int W, float eps,
                           float mult, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(add_sln_k<E>, dim3(T), dim3(256), 0, st, x, (const E*)y, (const E*)w, (E*)xa, W,
                                       eps, mult));
}

void layer_norm(bool bf16, const float* x, const void* w, void* out, int T, int W, float eps, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(layer_norm_k<E>, dim3(T), dim3(256), 0, st, x, (const E*)w, (E*)out, W, eps));
}

void rope_rows(bool bf16, void* q, int T, int H, int Dh, int offset, const float* table, int max_pos, int dims,
               const int64_t* pos, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(rope_rows_k<E>, dim3(T), dim3(256), 0, st, (E*)q, H, Dh, offset, table, max_pos,
                                       dims, pos));
}

void latent_kv_store(bool bf16, const void* dkv, int64_t ld, const void* norm_w, float eps, int rank, int rot_dim,
                     const float* table, int max_pos, int dims, const int64_t* pos, const int64_t* slots, void* rows,
                     int64_t num_rows, int T, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(latent_kv_store_k<E>, dim3(T), dim3(128), 0, st, (const E*)dkv, ld,
                                       (const E*)norm_w, eps, rank, rot_dim, table, max_pos, dims, pos, slots, (E*)rows,
                                       num_rows));
}

static int pad_row(int D, int esz) {
  // row stride (elements) whose dword stride is odd: lanes reading one column of 64 rows hit 64 banks
  if (esz == 4) return (D & 1) ? D : D + 1;
  int dp = (D + 1) & ~1;                   // even element count -> whole dwords
  return ((dp / 2) & 1) ? dp : dp + 2;
}

int latent_attention_plan(bool bf16, int H, int r, int dr, int* kt, int* nw) {
  const int esz = bf16 ? 2 : 4, D = r + dr;
  const int DP = pad_row(D, esz);
  const size_t qbytes = ((size_t)HB * D * 4 + 15) & ~(size_t)15;
  static const int opts[][2] = {{64, 4}, {64, 2}, {32, 4}, {32, 2}, {64, 1}, {16, 4}, {32, 1}, {16, 2}, {16, 1}};
  for (auto& o : opts) {
    const size_t wave = ((size_t)o[0] * DP * esz + (size_t)HB * o[0] * 4 + 15) & ~(size_t)15;
    if (wave < (size_t)HB * (r + 2) * 4) continue;
    const size_t total = qbytes + wave * o[1];
    if (total <= 64 * 1024) {
      *kt = o[0];
      *nw = o[1];
      return (int)total;
    }
  }
  return -1;
}

void latent_attention(bool bf16, const void* q_lat, const void* q_rot, int64_t qr_st, int64_t qr_sh, const void* rows,
                      int bs, const int32_t* block_tables, int bt_width, const int32_t* seq_of, const int64_t* pos,
                      float scale, const void* gate, int64_t g_st, void* out, int T, int H, int r, int dr,
                      hipStream_t st) {
  if (T <= 0) return;
  int KT = 0, NW = 0;
  const int lds = latent_attention_plan(bf16, H, r, dr, &KT, &NW);
  if (lds < 0) return;                     // refused by the caller beforehand
  const int DP = pad_row(r + dr, bf16 ? 2 : 4);
  const int rc = (r + 63) / 64;
  dim3 grid(T, (H + HB - 1) / HB), block(64 * NW);
#define SM_ATTN(RC)                                                                                                  \
  SM_DISPATCH(bf16, hipLaunchKernelGGL((latent_attn_k<E, RC>), grid, block, lds, st, (const E*)q_lat, (const E*)q_rot, \
                                       qr_st, qr_sh, (const E*)rows, bs, block_tables, bt_width, seq_of, pos, scale,   \
                                       (const E*)gate, g_st, (E*)out, H, r, dr, KT, DP))
  if (rc <= 1) { SM_ATTN(1); }
  else if (rc <= 2) { SM_ATTN(2); }
  else if (rc <= 4) { SM_ATTN(4); }
  else { SM_ATTN(8); }
#undef SM_ATTN
}

void mlstm_scan(bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                const void* ipre, int64_t i_ld, const void* fpre, int64_t f_ld, const float* ib, const float* fb,
                float cap, float* S, float* n, float* m, const int32_t* cu, const int32_t* slots, const int64_t* pos,
                float* out, int B, int H, int d, int dv, hipStream_t st) {
  if (B <= 0) return;
  const size_t lds = ((size_t)d * 64 + 3 * (size_t)d) * 4;
  dim3 grid(B, H, (dv + 63) / 64);
  SM_DISPATCH(bf16, hipLaunchKernelGGL(mlstm_scan_k<E>, grid, dim3(64), lds, st, (const E*)q, q_ld, (const E*)k, k_ld,
                                       (const E*)v, v_ld, (const E*)ipre, i_ld, (const E*)fpre, f_ld, ib, fb, cap, S, n,
                                       m, cu, slots, pos, out, H, d, dv));
}

void head_rms_gate(bool bf16, const float* h, const void* norm_w, const void* gate, int64_t g_ld, void* out, int T,
                   int H, int dv, float eps, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(head_rms_gate_k<E>, dim3(T, H), dim3(64), 0, st, h, (const E*)norm_w,
                                       (const E*)gate, g_ld, (E*)out, H, dv, eps));
}

void glu_gelu(bool bf16, const void* gu, void* out, int64_t T, int64_t I, hipStream_t st) {
  const int64_t n = T * I;
  if (n <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(glu_gelu_k<E>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                                       (const E*)gu, (E*)out, T, I));
}

}  // namespace sm
}  // namespace illm
