// Grouped-query attention with mixed head scores over paged [keys | values]
// rows (gfx950, wave64).
//
//   qk_norm_rope_store_k   per-head RMS norm + half-split rotary positions on
//                          queries and keys, cache append of [normed rotated
//                          keys | keys as projected]; queries leave in f32
//   talk_attn_k            one workgroup per (query token, key split): all H
//                          heads of the token together, because the scores of
//                          all heads at a key are mixed by an [H, H] matrix
//                          before the softmax.  Per key tile: scores (f32);
//                          mixing, causal mask and online softmax (16 lanes
//                          per head); weighted sum of the values (f32
//                          accumulators in registers).
//   talk_attn_combine_k    merge of the key splits + sigmoid output gate
//   talk_softmax_k         the scale + mixing + mask + softmax step of the
//                          library-product path of long portions
//
// Cache rows are bf16 or f32 (template E); queries, scores and weights are f32.
#include "blockmix.h"

#include <math.h>

namespace illm {
namespace bm {
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
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ------------------------------------------------------------------ norm + rotary + cache append
// one block per token, one wave per head in turn (query heads, then key heads); buf: (waves) x d floats
template <typename E>
__global__ void __launch_bounds__(1024) qk_norm_rope_store_k(const E* __restrict__ q, int64_t q_ld, const E* __restrict__ k,
                                                           int64_t k_ld, const E* __restrict__ qn, const E* __restrict__ kn,
                                                           float eps, const float* __restrict__ table, int max_pos,
                                                           int dims, const int64_t* __restrict__ pos,
                                                           const int64_t* __restrict__ slots, E* __restrict__ rows,
                                                           int64_t num_rows, float* __restrict__ qo, int H, int G, int d) {
  extern __shared__ float buf_all[];
  const int64_t t = blockIdx.x;
  const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* buf = buf_all + wv * d;
  int64_t p = pos[t];
  const bool in_table = p >= 0 && p < max_pos;
  if (!in_table) p = 0;
  const float* cs = table + p * dims;               // [dims / 2][2]
  const int half = dims >> 1;
  const int64_t slot = slots[t];
  const bool store = slot >= 0 && slot < num_rows;
  const int nwv = blockDim.x >> 6;
  for (int hh = wv; hh < H + G; hh += nwv) {
    const bool isq = hh < H;
    const E* src = isq ? q + t * q_ld + (int64_t)hh * d : k + t * k_ld + (int64_t)(hh - H) * d;
    const E* nw = isq ? qn : kn;
    float ss = 0.f;
    for (int i = lane; i < d; i += 64) {
      const float v = ldf(src + i);
      ss += v * v;
    }
    const float rs = nw ? 1.0f / sqrtf(wave_sum(ss) / (float)d + eps) : 1.0f;
    for (int i = lane; i < d; i += 64) buf[i] = ldf(src + i) * rs * (nw ? ldf(nw + i) : 1.0f);
    wave_sync();
    E* krow = store ? rows + slot * (int64_t)(2 * G * d) + (int64_t)(hh - H) * d : nullptr;
    for (int i = lane; i < d; i += 64) {
      float v = buf[i];
      if (i < dims && in_table) {
        const int j = i < half ? i : i - half;
        const float c = cs[2 * j], s = cs[2 * j + 1];
        v = i < half ? buf[i] * c - buf[i + half] * s : buf[i] * c + buf[i - half] * s;
      }
      if (isq) qo[(t * H + hh) * d + i] = v;
      else if (krow) {
        stf(krow + i, v);
        krow[(int64_t)G * d + i] = src[i];
      }
    }
    wave_sync();
  }
}

// ------------------------------------------------------------------ flash kernel
constexpr int kMaxItems = 4;        // (kv head, value column) items per thread: G d <= 1024

template <typename E> struct Words;   // a 4-byte word of cache row
template <> struct Words<float> {
  static constexpr int per = 1;
  static __device__ __forceinline__ void get(uint32_t w, float* v) { v[0] = __uint_as_float(w); }
};
template <> struct Words<__bf16> {
  static constexpr int per = 2;
  static __device__ __forceinline__ void get(uint32_t w, float* v) {
    v[0] = __uint_as_float(w << 16);
    v[1] = __uint_as_float(w & 0xffff0000u);
  }
};

typedef __bf16 bm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float bm_f32x4 __attribute__((ext_vector_type(4)));

__host__ __device__ __forceinline__ int round4(int n) { return (n + 3) & ~3; }

// LDS layout (floats unless noted, every region a multiple of 16 bytes): qs [H (d + 8)] | tk [H H] | S [H (KT + 1)] |
// S2 [H (KT + 1)] | mrun lrun corr [3 H] | red [JS H d] | tile (uint32 words) [KT pitch_w].
// MF (bf16 rows, d a multiple of 32): the scores run on the matrix cores -- 16 keys x 16 (padded) heads of one
// key / value head per 16x16x32 MFMA, the f32 queries split into bf16 hi + lo halves (qs then holds those, rows of
// d + 8) -- and the tile rows are 16-byte aligned; otherwise vector FMAs over rows of an odd word pitch.
template <typename E, int REP, bool MF>
__global__ void __launch_bounds__(256) talk_attn_k(const float* __restrict__ q, const E* __restrict__ rows, int bs,
                                                  const int32_t* __restrict__ block_tables, int bt_width,
                                                  const int32_t* __restrict__ seq_of, const int64_t* __restrict__ pos,
                                                  float scale, const float* __restrict__ talk, const E* __restrict__ gate,
                                                  int64_t g_st, E* __restrict__ out, float* __restrict__ part, int nsplit,
                                                  int H, int G, int d, int KT) {
  extern __shared__ float lds[];
  const int t = blockIdx.x, sp = blockIdx.y, tid = threadIdx.x;
  const int wv = tid >> 6, lane = tid & 63;
  const int Hd = H * d, Gd = G * d, KP = KT + 1;
  const int JS = Gd >= 256 ? 1 : 256 / Gd;
  constexpr int per = Words<E>::per;
  const int row_w = 2 * Gd / per;                   // words per cache row
  const int pitch = MF ? row_w + 4 : (row_w | 1);   // aligned rows for MFMA operands, else an odd word pitch
  const int DP = d + 8;
  float* qs = lds;
  float* tk = qs + round4(H * DP);
  float* S = tk + round4(H * H);
  float* S2 = S + round4(H * KP);
  float* mrun = S2 + round4(H * KP);
  float* lrun = mrun + H;
  float* corr = lrun + H;
  float* red = mrun + round4(3 * H);
  uint32_t* tile = (uint32_t*)(red + round4(JS * Hd));

  const int64_t L = pos[t] + 1;                     // keys this token sees
  const int b = seq_of[t];
  const int32_t* bt = block_tables + (int64_t)b * bt_width;
  const int64_t tiles_total = (L + KT - 1) / KT;
  const int64_t tiles_per = (tiles_total + nsplit - 1) / nsplit;
  const int64_t k_lo = (int64_t)sp * tiles_per * KT;
  const int64_t k_hi = L < k_lo + tiles_per * KT ? L : k_lo + tiles_per * KT;

  if (MF) {
    __bf16* qh = (__bf16*)qs;
    __bf16* ql = qh + H * DP;
    for (int i = tid; i < Hd; i += 256) {
      const int h = i / d, c = i - h * d;
      const float v = q[(int64_t)t * Hd + i];
      const __bf16 hi = (__bf16)v;
      qh[h * DP + c] = hi;
      ql[h * DP + c] = (__bf16)(v - (float)hi);
    }
  } else {
    for (int i = tid; i < Hd; i += 256) qs[i] = q[(int64_t)t * Hd + i];
  }
  for (int i = tid; i < H * H; i += 256) tk[i] = talk ? talk[i] : ((i / H) == (i % H) ? 1.f : 0.f);
  if (tid < H) {
    mrun[tid] = -INFINITY;
    lrun[tid] = 0.f;
    corr[tid] = 0.f;
  }
  float acc[kMaxItems][REP];
#pragma unroll
  for (int a = 0; a < kMaxItems; a++)
#pragma unroll
    for (int r = 0; r < REP; r++) acc[a][r] = 0.f;
  const int js = JS > 1 ? tid / Gd : 0;
  const bool pv_on = JS > 1 ? tid < JS * Gd : true;
  __syncthreads();

  // MF: a tile's rows lie in one page, one after the other (KT divides the page size), so the tile is one run of
  // 16-byte pieces; the next tile's pieces are requested before the current tile's arithmetic
  constexpr int kMaxPre = MF ? 8 : 1;
  uint4 pre[kMaxPre];
  const int npiece = KT * (row_w / 4);
  auto request = [&](int64_t j0) {
    const int nvr = (int)(k_hi - j0 < KT ? k_hi - j0 : KT);
    const uint4* src = (const uint4*)((const uint32_t*)rows + ((int64_t)bt[j0 / bs] * bs + j0 % bs) * row_w);
#pragma unroll
    for (int it = 0; it < kMaxPre; it++) {
      const int i = tid + 256 * it;
      pre[it] = make_uint4(0u, 0u, 0u, 0u);
      if (i < npiece && i / (row_w / 4) < nvr) pre[it] = src[i];
    }
  };
  if (MF && k_lo < k_hi) request(k_lo);
  for (int64_t j0 = k_lo; j0 < k_hi; j0 += KT) {
    const int nv = (int)(k_hi - j0 < KT ? k_hi - j0 : KT);
    if (MF) {
#pragma unroll
      for (int it = 0; it < kMaxPre; it++) {
        const int i = tid + 256 * it;
        if (i < npiece && i / (row_w / 4) < nv) {
          const int j = i / (row_w / 4), c = i - j * (row_w / 4);
          *(uint4*)(tile + j * pitch + c * 4) = pre[it];
        }
      }
      __syncthreads();
      if (j0 + KT < k_hi) request(j0 + KT);
    } else {
    // ---- tile load: 16-byte pieces of the nv rows
    {
      const int pieces = row_w / 4;                 // row_w is a multiple of 4 words (d % 8 == 0)
      for (int i = tid; i < nv * pieces; i += 256) {
        const int j = i / pieces, c = i - j * pieces;
        const int64_t kp = j0 + j;
        const int64_t row = (int64_t)bt[kp / bs] * bs + kp % bs;
        const uint4 v = *(const uint4*)((const uint32_t*)rows + row * row_w + c * 4);
        uint32_t* dst = tile + j * pitch + c * 4;
        dst[0] = v.x;
        dst[1] = v.y;
        dst[2] = v.z;
        dst[3] = v.w;
      }
    }
    __syncthreads();
    }
    // ---- scores
    if (MF) {
      const int r16 = lane & 15, gq = lane >> 4;
      const __bf16* qh = (const __bf16*)qs;
      const __bf16* ql = qh + H * DP;
      const int nchunk = (nv + 15) >> 4;
      const bool hv = r16 < REP;
      const bm_bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
      for (int u = wv; u < G * nchunk; u += 4) {
        const int g = u / nchunk, kc = u - g * nchunk;
        const int h = g * REP + (hv ? r16 : 0);
        const __bf16* ka = (const __bf16*)tile + (int64_t)(kc * 16 + r16) * pitch * 2 + g * d + 8 * gq;
        const __bf16* qa = qh + h * DP + 8 * gq;
        const __bf16* qb = ql + h * DP + 8 * gq;
        bm_f32x4 a4 = {0.f, 0.f, 0.f, 0.f};
        for (int ks = 0; ks < d / 32; ks++) {
          const bm_bf16x8 a = *(const bm_bf16x8*)(ka + 32 * ks);
          const bm_bf16x8 bh = hv ? *(const bm_bf16x8*)(qa + 32 * ks) : zero8;
          const bm_bf16x8 bl = hv ? *(const bm_bf16x8*)(qb + 32 * ks) : zero8;
          a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bh, a4, 0, 0, 0);
          a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bl, a4, 0, 0, 0);
        }
        if (hv) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int key = kc * 16 + 4 * gq + i;     // lane: keys 4 gq + i of head r16
            if (key < KT) S[h * KP + key] = a4[i] * scale;
          }
        }
      }
    } else
    for (int it = tid; it < KT * G; it += 256) {
      const int j = it % KT, g = it / KT;
      if (j < nv) {
        float a[REP];
#pragma unroll
        for (int r = 0; r < REP; r++) a[r] = 0.f;
        const uint32_t* kr = tile + j * pitch + g * d / per;
        const float* qg = qs + g * REP * d;
        for (int i = 0; i < d / per; i++) {
          float kv[2];
          Words<E>::get(kr[i], kv);
#pragma unroll
          for (int r = 0; r < REP; r++) {
#pragma unroll
            for (int e = 0; e < per; e++) a[r] += qg[r * d + i * per + e] * kv[e];
          }
        }
#pragma unroll
        for (int r = 0; r < REP; r++) S[(g * REP + r) * KP + j] = a[r] * scale;
      }
    }
    __syncthreads();
    // ---- mixing over the heads, mask and online softmax in one phase: 16 lanes per head (four heads per wave
    // at a time), lane gl takes keys gl, gl + 16, ...; the weights go to S2 (S is still read by the other heads)
    {
      const int gl = lane & 15, hq = lane >> 4;
      for (int h0 = wv * 4; h0 < H; h0 += 16) {
        const int h = h0 + hq;
        if (h < H) {
          float sj[4];
          float mt = -INFINITY;
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const int j = gl + 16 * u;
            float v = -INFINITY;
            if (j < nv) {
              v = 0.f;
              for (int g = 0; g < H; g++) v += tk[h * H + g] * S[g * KP + j];
            }
            sj[u] = v;
            mt = fmaxf(mt, v);
          }
#pragma unroll
          for (int o = 8; o > 0; o >>= 1) mt = fmaxf(mt, __shfl_xor(mt, o, 64));
          const float mo = mrun[h], mn = fmaxf(mo, mt);
          float ls = 0.f;
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const int j = gl + 16 * u;
            const float pj = sj[u] == -INFINITY ? 0.f : expf(sj[u] - mn);
            if (j < KT) S2[h * KP + j] = pj;
            ls += pj;
          }
#pragma unroll
          for (int o = 8; o > 0; o >>= 1) ls += __shfl_xor(ls, o, 64);
          if (gl == 0) {
            const float c = expf(mo - mn);            // mo = -inf at the first tile: 0
            corr[h] = c;
            lrun[h] = lrun[h] * c + ls;
            mrun[h] = mn;
          }
        }
      }
    }
    __syncthreads();
    // ---- weighted sum of the values
    if (pv_on) {
#pragma unroll
      for (int a = 0; a < kMaxItems; a++) {
        const int item = JS > 1 ? tid - js * Gd : tid + a * 256;
        if ((JS > 1 && a > 0) || item >= Gd) break;
        const int g = item / d;
#pragma unroll
        for (int r = 0; r < REP; r++) acc[a][r] *= corr[g * REP + r];
        const E* vcol = (const E*)tile + Gd + item;
        for (int j = js; j < nv; j += JS) {
          const float v = ldf(vcol + (int64_t)j * pitch * per);
#pragma unroll
          for (int r = 0; r < REP; r++) acc[a][r] += S2[(g * REP + r) * KP + j] * v;
        }
      }
    }
    __syncthreads();
  }
  // ---- partial sums of the key-interleaved thread groups -> red [JS][H d]
  if (pv_on) {
#pragma unroll
    for (int a = 0; a < kMaxItems; a++) {
      const int item = JS > 1 ? tid - js * Gd : tid + a * 256;
      if ((JS > 1 && a > 0) || item >= Gd) break;
      const int g = item / d, c = item - g * d;
#pragma unroll
      for (int r = 0; r < REP; r++) red[js * Hd + (g * REP + r) * d + c] = acc[a][r];
    }
  }
  __syncthreads();
  for (int o = tid; o < Hd; o += 256) {
    const int h = o / d, c = o - h * d;
    float v = 0.f;
    for (int s = 0; s < JS; s++) v += red[s * Hd + o];
    if (nsplit == 1) {
      v /= lrun[h];
      if (gate) v *= 1.0f / (1.0f + expf(-ldf(gate + (int64_t)t * g_st + o)));
      stf(out + (int64_t)t * Hd + o, v);
    } else {
      float* pr = part + (((int64_t)t * nsplit + sp) * H + h) * (d + 2);
      pr[c] = v;
      if (c == 0) {
        pr[d] = mrun[h];
        pr[d + 1] = lrun[h];
      }
    }
  }
}

// one block per (token, head): the splits' maxima and sums by the first wave, then a thread per value column
template <typename E>
__global__ void __launch_bounds__(128) talk_attn_combine_k(const float* __restrict__ part, const E* __restrict__ gate,
                                                          int64_t g_st, E* __restrict__ out, int nsplit, int H, int d) {
  __shared__ float wgt[64];
  __shared__ float linv;
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, tid = threadIdx.x;
  const float* pr = part + ((int64_t)t * nsplit * H + h) * (d + 2);
  const int64_t st = (int64_t)H * (d + 2);
  if (tid < 64) {
    const float m = tid < nsplit ? pr[tid * st + d] : -INFINITY;
    const float M = wave_max(m);
    const float e = m == -INFINITY ? 0.f : expf(m - M);       // an empty split weighs nothing
    const float l = wave_sum(tid < nsplit ? pr[tid * st + d + 1] * e : 0.f);
    wgt[tid] = e;
    if (tid == 0) linv = 1.0f / l;
  }
  __syncthreads();
  for (int c = tid; c < d; c += 128) {
    float v = 0.f;
    for (int s = 0; s < nsplit; s++) v += pr[s * st + c] * wgt[s];
    v *= linv;
    const int o = h * d + c;
    if (gate) v *= 1.0f / (1.0f + expf(-ldf(gate + t * g_st + o)));
    stf(out + t * (int64_t)H * d + o, v);
  }
}

// ------------------------------------------------------------------ long portions on the matrix cores (bf16 rows)
// One workgroup of NW waves per 16 consecutive query tokens of one sequence's portion, all H = NW HW heads; wave w owns heads
// w HW .. w HW + HW - 1 (their query fragments, split into bf16 hi + lo halves, and their output accumulators stay in
// registers).  Per tile of 16 keys: the cache rows as they are into LDS; scores as 16x16x32 MFMAs (D[key][token]);
// mixing over the heads as one small MFMA product per token (matrix and scores as bf16 hi + lo halves) with the
// causal mask; online softmax by one thread per (head, token) row, weights written as bf16 hi + lo; weighted sums as 16x16x16 MFMAs (D[token][column]) whose value
// operand a lane gathers from four rows (16 lanes read 32 contiguous bytes, the four row groups fall into other banks).
typedef short bm_s16x4 __attribute__((ext_vector_type(4)));
constexpr int PF_KT = 16, PF_SP = PF_KT + 4, PF_PP = PF_KT + 4;

__host__ __device__ __forceinline__ int pf_lds_bytes(int H, int G, int d) {
  const int Gd = G * d;
  return 4 * (round4(H * H) + H * 16 * PF_SP + 2 * round4(H * 16)) + 2 * (PF_KT * (2 * Gd + 8) + 2 * H * 16 * PF_PP);
}

template <int D16, int HW, int NW>
__global__ void __launch_bounds__(64 * NW) talk_prefill_k(const float* __restrict__ q, const __bf16* __restrict__ rows, int bs,
                                                     const int32_t* __restrict__ bt, const int64_t* __restrict__ pos,
                                                     int t0, int n, float scale, const float* __restrict__ talk,
                                                     const __bf16* __restrict__ gate, int64_t g_st,
                                                     __bf16* __restrict__ out, int G, float* __restrict__ part,
                                                     int nsplit) {
  constexpr int H = NW * HW, d = 16 * D16, KS = D16 / 2, NT = 64 * NW, TPW = 16 / NW;
  extern __shared__ float lds[];
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, r16 = lane & 15, gq = lane >> 4;
  const int Gd = G * d, REP = H / G, KP = 2 * Gd + 8;
  float* tk = lds;
  float* S = tk + round4(H * H);
  float* corr = S + H * 16 * PF_SP;
  float* linv = corr + round4(H * 16);
  __bf16* Kt = (__bf16*)(linv + round4(H * 16));
  __bf16* Ph = Kt + PF_KT * KP;
  __bf16* Pl = Ph + H * 16 * PF_PP;

  const int tq0 = t0 + 16 * (gridDim.x - 1 - blockIdx.x);     // first token of this tile; the longest tiles start first
  const int nq = t0 + n - tq0 < 16 ? t0 + n - tq0 : 16;       // valid tokens
  const int64_t p0 = pos[tq0];                                // consecutive positions p0 .. p0 + nq - 1
  // key splits (blockIdx.y): whole 16-key tiles of the keys the tile's last token sees; a split past them is empty
  const int64_t tiles_total = (p0 + nq + PF_KT - 1) / PF_KT, tiles_per = (tiles_total + nsplit - 1) / nsplit;
  const int64_t k_lo = (int64_t)blockIdx.y * tiles_per * PF_KT;
  const int64_t nkeys = p0 + nq < k_lo + tiles_per * PF_KT ? p0 + nq : k_lo + tiles_per * PF_KT;

  // query fragments: lane (token r16, k part gq) of every owned head
  bm_bf16x8 qh[HW][KS], ql[HW][KS];
#pragma unroll
  for (int hh = 0; hh < HW; hh++) {
    const int h = wv * HW + hh;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const float* src = q + ((int64_t)(tq0 + (r16 < nq ? r16 : 0)) * H + h) * d + 32 * ks + 8 * gq;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float v = r16 < nq ? src[e] : 0.f;
        const __bf16 hi = (__bf16)v;
        qh[hh][ks][e] = hi;
        ql[hh][ks][e] = (__bf16)(v - (float)hi);
      }
    }
  }
  bm_s16x4 th = {0, 0, 0, 0}, tl = {0, 0, 0, 0};               // mixing matrix: lane (head r16, g part gq)
  if (talk) {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int g = 4 * gq + e;
      const float v = (r16 < H && g < H) ? talk[r16 * H + g] : 0.f;
      const __bf16 hi = (__bf16)v;
      th[e] = __builtin_bit_cast(short, hi);
      tl[e] = __builtin_bit_cast(short, (__bf16)(v - (float)hi));
    }
  }
  bm_f32x4 acc[HW][D16];
#pragma unroll
  for (int hh = 0; hh < HW; hh++)
#pragma unroll
    for (int nt = 0; nt < D16; nt++) acc[hh][nt] = bm_f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;                       // of row tid = (head tid / 16, token tid % 16)
  const int pieces = Gd / 8;
  const bm_bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // a tile's 16 rows lie in one page, one after the other: 16-byte pieces tid, tid + 256, ... of that run.  The next
  // tile's pieces are requested before the current tile's arithmetic and land in LDS after it.
  constexpr int kMaxNL = 2048 / NT;                           // 2 G d <= 1024
  const int npiece = PF_KT * pieces * 2;
  bm_bf16x8 pre[kMaxNL];
  auto request = [&](int64_t j0) {
    const int nvr = (int)(nkeys - j0 < PF_KT ? nkeys - j0 : PF_KT);
    const __bf16* src = rows + ((int64_t)bt[j0 / bs] * bs + j0 % bs) * 2 * Gd;
#pragma unroll
    for (int it = 0; it < kMaxNL; it++) {
      const int i = tid + NT * it;
      pre[it] = zero8;
      if (i < npiece && i / (2 * pieces) < nvr) pre[it] = *(const bm_bf16x8*)(src + (int64_t)i * 8);
    }
  };
  if (k_lo < nkeys) request(k_lo);
  for (int64_t j0 = k_lo; j0 < nkeys; j0 += PF_KT) {
    const int nv = (int)(nkeys - j0 < PF_KT ? nkeys - j0 : PF_KT);
    // ---- the tile's rows [keys | values]; rows past nv are zero
#pragma unroll
    for (int it = 0; it < kMaxNL; it++) {
      const int i = tid + NT * it;
      if (i < npiece) {
        const int j = i / (2 * pieces), c = i - j * 2 * pieces;
        *(bm_bf16x8*)(Kt + j * KP + c * 8) = pre[it];
      }
    }
    __syncthreads();
    if (j0 + PF_KT < nkeys) request(j0 + PF_KT);
    // ---- scores: D[key 4 gq + i][token r16] of every owned head
#pragma unroll
    for (int hh = 0; hh < HW; hh++) {
      const int h = wv * HW + hh, g = h / REP;
      const __bf16* ka = Kt + r16 * KP + g * d + 8 * gq;
      bm_f32x4 a4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const bm_bf16x8 a = *(const bm_bf16x8*)(ka + 32 * ks);
        a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qh[hh][ks], a4, 0, 0, 0);
        a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ql[hh][ks], a4, 0, 0, 0);
      }
      *(float4*)(S + (h * 16 + r16) * PF_SP + 4 * gq) = make_float4(a4[0] * scale, a4[1] * scale, a4[2] * scale, a4[3] * scale);
    }
    __syncthreads();
    // ---- mixing over the heads + causal mask: wave w takes 16 / NW tokens; per token one 16 x 16 x 16
    // product D[head][key] = T[head][g] S[g][key], T and S as bf16 hi + lo halves (hi hi + hi lo + lo hi)
#pragma unroll
    for (int tt = 0; tt < TPW; tt++) {
      const int t = wv * TPW + tt;
      const bool vis = t < nq && r16 < nv && j0 + r16 <= p0 + t;
      if (talk) {
        bm_s16x4 bh, bl;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int g = 4 * gq + e;
          const float v = g < H ? S[(g * 16 + t) * PF_SP + r16] : 0.f;
          const __bf16 hi = (__bf16)v;
          bh[e] = __builtin_bit_cast(short, hi);
          bl[e] = __builtin_bit_cast(short, (__bf16)(v - (float)hi));
        }
        bm_f32x4 m4 = {0.f, 0.f, 0.f, 0.f};
        m4 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(th, bh, m4, 0, 0, 0);
        m4 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(th, bl, m4, 0, 0, 0);
        m4 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(tl, bh, m4, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (4 * gq + i < H) S[((4 * gq + i) * 16 + t) * PF_SP + r16] = vis ? m4[i] : -INFINITY;
      } else if (!vis) {
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (4 * gq + i < H) S[((4 * gq + i) * 16 + t) * PF_SP + r16] = -INFINITY;
      }
    }
    __syncthreads();
    // ---- online softmax: thread tid < 16 H owns row (head tid / 16, token tid % 16)
    if (tid < H * 16) {
      float sv[PF_KT];
#pragma unroll
      for (int c = 0; c < PF_KT / 4; c++) {
        const float4 v = *(const float4*)(S + tid * PF_SP + 4 * c);
        sv[4 * c] = v.x; sv[4 * c + 1] = v.y; sv[4 * c + 2] = v.z; sv[4 * c + 3] = v.w;
      }
      float mt = m_run;
#pragma unroll
      for (int j = 0; j < PF_KT; j++) mt = fmaxf(mt, sv[j]);
      const float c = mt == -INFINITY ? 1.f : __expf(m_run - mt);
      float ls = 0.f;
#pragma unroll
      for (int c4i = 0; c4i < PF_KT / 4; c4i++) {
        bm_s16x4 hi4, lo4;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float sj = sv[4 * c4i + e];
          const float pj = sj == -INFINITY ? 0.f : __expf(sj - mt);
          ls += pj;
          const __bf16 hi = (__bf16)pj;
          const __bf16 lo = (__bf16)(pj - (float)hi);
          hi4[e] = __builtin_bit_cast(short, hi);
          lo4[e] = __builtin_bit_cast(short, lo);
        }
        *(bm_s16x4*)(Ph + tid * PF_PP + 4 * c4i) = hi4;
        *(bm_s16x4*)(Pl + tid * PF_PP + 4 * c4i) = lo4;
      }
      l_run = l_run * c + ls;
      m_run = mt;
      corr[tid] = c;
    }
    __syncthreads();
    // ---- weighted sums: D[token 4 gq + i][column r16] of every owned head and column tile
    {
      float4 c4[HW];
      bm_s16x4 ah[HW], al[HW];
#pragma unroll
      for (int hh = 0; hh < HW; hh++) {
        const int h = wv * HW + hh;
        c4[hh] = *(const float4*)(corr + h * 16 + 4 * gq);
        ah[hh] = *(const bm_s16x4*)(Ph + (h * 16 + r16) * PF_PP + 4 * gq);
        al[hh] = *(const bm_s16x4*)(Pl + (h * 16 + r16) * PF_PP + 4 * gq);
      }
      bool moved = false;
#pragma unroll
      for (int hh = 0; hh < HW; hh++)
        moved |= c4[hh].x != 1.f || c4[hh].y != 1.f || c4[hh].z != 1.f || c4[hh].w != 1.f;
      if (__any(moved)) {                             // some running maximum of this wave's rows grew
#pragma unroll
        for (int hh = 0; hh < HW; hh++)
#pragma unroll
          for (int nt = 0; nt < D16; nt++) {
            acc[hh][nt][0] *= c4[hh].x;
            acc[hh][nt][1] *= c4[hh].y;
            acc[hh][nt][2] *= c4[hh].z;
            acc[hh][nt][3] *= c4[hh].w;
          }
      }
      const short* vbase = (const short*)Kt + (4 * gq) * KP + Gd + r16;
#pragma unroll
      for (int nt = 0; nt < D16; nt++) {
        bm_s16x4 b = {0, 0, 0, 0};
        int gprev = -1;
#pragma unroll
        for (int hh = 0; hh < HW; hh++) {
          const int g = (wv * HW + hh) / REP;
          if (g != gprev) {                           // keys 4 gq .. 4 gq + 3 at column nt 16 + r16 of value head g
            const short* vb = vbase + g * d + nt * 16;
            b[0] = vb[0];
            b[1] = vb[KP];
            b[2] = vb[2 * KP];
            b[3] = vb[3 * KP];
            gprev = g;
          }
          bm_f32x4 a = acc[hh][nt];
          a = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ah[hh], b, a, 0, 0, 0);
          a = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(al[hh], b, a, 0, 0, 0);
          acc[hh][nt] = a;
        }
      }
    }
    __syncthreads();
  }
  if (nsplit > 1) {
    // unnormalised sums, running maximum and sum of every (token, head) row: merged by talk_attn_combine_k
    if (tid < H * 16 && (tid & 15) < nq) {
      float* pr = part + (((int64_t)(tq0 - t0 + (tid & 15)) * nsplit + blockIdx.y) * H + (tid >> 4)) * (d + 2);
      pr[d] = m_run;
      pr[d + 1] = l_run;
    }
#pragma unroll
    for (int hh = 0; hh < HW; hh++) {
      const int h = wv * HW + hh;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int t = 4 * gq + i;
        if (t >= nq) continue;
        float* pr = part + (((int64_t)(tq0 - t0 + t) * nsplit + blockIdx.y) * H + h) * (d + 2);
#pragma unroll
        for (int nt = 0; nt < D16; nt++) pr[nt * 16 + r16] = acc[hh][nt][i];
      }
    }
    return;
  }
  if (tid < H * 16) linv[tid] = 1.0f / l_run;
  __syncthreads();
#pragma unroll
  for (int hh = 0; hh < HW; hh++) {
    const int h = wv * HW + hh;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int t = 4 * gq + i;
      if (t >= nq) continue;
      const float li = linv[h * 16 + t];
      const int64_t tq = tq0 + t;
#pragma unroll
      for (int nt = 0; nt < D16; nt++) {
        const int o = h * d + nt * 16 + r16;
        float v = acc[hh][nt][i] * li;
        if (gate) v *= 1.0f / (1.0f + expf(-(float)gate[tq * g_st + o]));
        out[tq * (int64_t)H * d + o] = (__bf16)v;
      }
    }
  }
}

// ------------------------------------------------------------------ softmax step of the library-product path
// one block per token: rows t H .. t H + H - 1 of sc [nt H, L].  Pass A mixes the H raw scores of every key
// column (scaled) in place; pass B is the masked softmax of every row, a wave per row in turn.
template <typename E, int HM>
__global__ void __launch_bounds__(256) talk_softmax_k(float* __restrict__ sc, const int64_t* __restrict__ pos, int H,
                                                     float scale, const float* __restrict__ talk, int L,
                                                     E* __restrict__ hi, E* __restrict__ lo) {
  __shared__ float tk[HM * HM];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
  float* base = sc + t * H * (int64_t)L;
  int64_t nk = pos[t] + 1;
  if (nk > L) nk = L;
  if (nk < 0) nk = 0;
  if (talk) {
    for (int i = tid; i < H * H; i += 256) tk[i] = talk[i] * scale;
    __syncthreads();
    for (int j = tid; j < nk; j += 256) {
      float s[HM];
#pragma unroll
      for (int g = 0; g < HM; g++) s[g] = g < H ? base[(int64_t)g * L + j] : 0.f;
#pragma unroll
      for (int h = 0; h < HM; h++) {
        if (h < H) {
          float v = 0.f;
#pragma unroll
          for (int g = 0; g < HM; g++)
            if (g < H) v += tk[h * H + g] * s[g];
          base[(int64_t)h * L + j] = v;
        }
      }
    }
    __syncthreads();
  }
  const float post = talk ? 1.0f : scale;
  for (int h = wv; h < H; h += 4) {
    float* r = base + (int64_t)h * L;
    float m = -INFINITY;
    for (int j = lane; j < nk; j += 64) m = fmaxf(m, r[j] * post);
    m = wave_max(m);
    float l = 0.f;
    for (int j = lane; j < nk; j += 64) l += expf(r[j] * post - m);
    l = wave_sum(l);
    const float inv = 1.0f / l;
    for (int j = lane; j < L; j += 64) {
      const float p = j < nk ? expf(r[j] * post - m) * inv : 0.f;
      if (hi) {
        const __bf16 ph = (__bf16)p;
        const int64_t o = (t * H + h) * (int64_t)L + j;
        ((__bf16*)hi)[o] = ph;
        ((__bf16*)lo)[o] = (__bf16)(p - (float)ph);
      } else {
        r[j] = p;
      }
    }
  }
}

int lds_floats(int H, int G, int d, int KT) {
  const int Gd = G * d, JS = Gd >= 256 ? 1 : 256 / Gd;
  return round4(H * (d + 8)) + round4(H * H) + 2 * round4(H * (KT + 1)) + round4(3 * H) + round4(JS * H * d);
}

bool use_mfma(bool bf16, int d) { return bf16 && d % 32 == 0; }

}  // namespace

void qk_norm_rope_store(bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* qn,
                        const void* kn, float eps, const float* table, int max_pos, int dims, const int64_t* pos,
                        const int64_t* slots, void* rows, int64_t num_rows, float* qo, int T, int H, int G, int d,
                        hipStream_t st) {
  if (T <= 0) return;
  int nwv = H + G >= 16 ? 16 : H + G;               // few rows: a wave per head, within 48 KB of LDS
  if (T > 64 && nwv > 4) nwv = 4;
  if (nwv * d > 12288) nwv = 12288 / d < 1 ? 1 : 12288 / d;
  const size_t lds = (size_t)nwv * d * sizeof(float);
  if (bf16)
    qk_norm_rope_store_k<__bf16><<<T, 64 * nwv, lds, st>>>((const __bf16*)q, q_ld, (const __bf16*)k, k_ld, (const __bf16*)qn,
                                                      (const __bf16*)kn, eps, table, max_pos, dims, pos, slots,
                                                      (__bf16*)rows, num_rows, qo, H, G, d);
  else
    qk_norm_rope_store_k<float><<<T, 64 * nwv, lds, st>>>((const float*)q, q_ld, (const float*)k, k_ld, (const float*)qn,
                                                     (const float*)kn, eps, table, max_pos, dims, pos, slots,
                                                     (float*)rows, num_rows, qo, H, G, d);
}

int talk_attention_plan(bool bf16, int H, int G, int d, int* kt) {
  if (H < 1 || G < 1 || H % G || d < 8 || d % 8 || G * d > 256 * kMaxItems) return -1;
  const int rep = H / G;
  if (rep > 8) return -1;
  const int per = bf16 ? 2 : 1;
  const bool mf = use_mfma(bf16, d);
  const int pitch = mf ? 2 * G * d / per + 4 : ((2 * G * d / per) | 1);
  for (int KT = 64; KT >= (mf ? 16 : 8); KT >>= 1) {
    const int64_t bytes = (int64_t)lds_floats(H, G, d, KT) * 4 + (int64_t)KT * pitch * 4;
    if (mf && (int64_t)KT * (2 * G * d / per) / 4 > 8 * 256) continue;       // the prefetch registers hold 8 pieces
    if (bytes <= 64 * 1024) {
      *kt = KT;
      return (int)bytes;
    }
  }
  return -1;
}

int talk_attention_splits(bool bf16, int T, int H, int G, int d, int max_ctx) {
  int kt = 0;
  if (talk_attention_plan(bf16, H, G, d, &kt) < 0) return 1;
  const int tiles = (max_ctx + kt - 1) / kt;
  int ns = 1;
  // fill the chip (256 CUs, a few workgroups each), at least 4 tiles per split
  while (ns < 64 && (int64_t)T * ns < 1024 && tiles / (ns * 2) >= 2) ns *= 2;
  return ns;
}

template <typename E, int REP, bool MF>
static void launch_talk(const float* q, const void* rows, int bs, const int32_t* bt, int btw, const int32_t* seq_of,
                        const int64_t* pos, float scale, const float* talk, const void* gate, int64_t g_st, void* out,
                        float* part, int nsplit, int T, int H, int G, int d, int KT, int lds, hipStream_t st) {
  talk_attn_k<E, REP, MF><<<dim3(T, nsplit), 256, lds, st>>>(q, (const E*)rows, bs, bt, btw, seq_of, pos, scale, talk,
                                                          (const E*)gate, g_st, (E*)out, part, nsplit, H, G, d, KT);
}

void talk_attention(bool bf16, const float* q, const void* rows, int bs, const int32_t* block_tables, int bt_width,
                    const int32_t* seq_of, const int64_t* pos, float scale, const float* talk, const void* gate,
                    int64_t g_st, void* out, float* part, int nsplit, int T, int H, int G, int d, hipStream_t st) {
  if (T <= 0) return;
  int KT = 0;
  const int lds = talk_attention_plan(bf16, H, G, d, &KT);
  if (lds < 0) return;                              // callers check the plan first
#define BM_REP(R)                                                                                                     \
  case R:                                                                                                             \
    if (bf16 && use_mfma(true, d))                                                                                    \
      launch_talk<__bf16, R, true>(q, rows, bs, block_tables, bt_width, seq_of, pos, scale, talk, gate, g_st, out,    \
                                   part, nsplit, T, H, G, d, KT, lds, st);                                            \
    else if (bf16)                                                                                                    \
      launch_talk<__bf16, R, false>(q, rows, bs, block_tables, bt_width, seq_of, pos, scale, talk, gate, g_st, out,   \
                                    part, nsplit, T, H, G, d, KT, lds, st);                                           \
    else launch_talk<float, R, false>(q, rows, bs, block_tables, bt_width, seq_of, pos, scale, talk, gate, g_st, out, part,  \
                               nsplit, T, H, G, d, KT, lds, st);                                                      \
    break;
  switch (H / G) {
    BM_REP(1) BM_REP(2) BM_REP(3) BM_REP(4) BM_REP(5) BM_REP(6) BM_REP(7) BM_REP(8)
    default: return;
  }
#undef BM_REP
  if (nsplit > 1) {
    if (bf16)
      talk_attn_combine_k<__bf16><<<dim3(T, H), 128, 0, st>>>(part, (const __bf16*)gate, g_st, (__bf16*)out, nsplit, H, d);
    else
      talk_attn_combine_k<float><<<dim3(T, H), 128, 0, st>>>(part, (const float*)gate, g_st, (float*)out, nsplit, H, d);
  }
}

bool talk_prefill_fits(int H, int G, int d) {
  return (H == 4 || H == 8 || H == 16) && (d == 64 || d == 128) && G >= 1 && H % G == 0 && G * d <= 512 &&
         pf_lds_bytes(H, G, d) <= 150 * 1024;
}

template <int D16, int HW, int NW>
static void launch_prefill(const float* q, const void* rows, int bs, const int32_t* bt, const int64_t* pos, int t0, int n,
                           float scale, const float* talk, const void* gate, int64_t g_st, void* out, int G, float* part,
                           int nsplit, hipStream_t st) {
  const int H = NW * HW, d = 16 * D16;
  const int lds = pf_lds_bytes(H, G, d);
  static int granted = 0;                             // dynamic LDS past 64 KB is granted per kernel
  if (lds > granted) {
    hipFuncSetAttribute((const void*)talk_prefill_k<D16, HW, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    granted = lds;
  }
  talk_prefill_k<D16, HW, NW><<<dim3((n + 15) / 16, nsplit), 64 * NW, lds, st>>>(
      q, (const __bf16*)rows, bs, bt, pos, t0, n, scale, talk, (const __bf16*)gate, g_st, (__bf16*)out, G, part, nsplit);
  if (nsplit > 1)
    talk_attn_combine_k<__bf16><<<dim3(n, H), 128, 0, st>>>(part, gate ? (const __bf16*)gate + (int64_t)t0 * g_st : nullptr,
                                                            g_st, (__bf16*)out + (int64_t)t0 * H * d, nsplit, H, d);
}

// key splits of a portion whose last token sees max_keys keys: the causal lengths of the 16-token tiles differ
// by a factor of two around their mean, so long portions are cut into more, shorter workgroups
int talk_prefill_splits(int n, int max_keys) {
  int ns = max_keys / 1024;
  return ns < 1 ? 1 : (ns > 4 ? 4 : ns);
}

void talk_prefill(const float* q, const void* rows, int bs, const int32_t* bt, const int64_t* pos, int t0, int n,
                  float scale, const float* talk, const void* gate, int64_t g_st, void* out, float* part, int nsplit,
                  int H, int G, int d, hipStream_t st) {
  if (n <= 0 || !talk_prefill_fits(H, G, d)) return;
#define BM_PF(D16, HW, NW) \
  launch_prefill<D16, HW, NW>(q, rows, bs, bt, pos, t0, n, scale, talk, gate, g_st, out, G, part, nsplit, st)
  if (d == 64) {
    if (H == 4) BM_PF(4, 1, 4); else if (H == 8) BM_PF(4, 2, 4); else BM_PF(4, 2, 8);
  } else {
    if (H == 4) BM_PF(8, 1, 4); else if (H == 8) BM_PF(8, 1, 8); else BM_PF(8, 2, 8);
  }
#undef BM_PF
}

void talk_softmax(bool bf16, float* sc, const int64_t* pos, int H, float scale, const float* talk, int64_t nt, int L,
                  void* hi, void* lo, hipStream_t st) {
  if (nt <= 0) return;
#define BM_HM(HM)                                                                                                  \
  if (bf16) talk_softmax_k<__bf16, HM><<<nt, 256, 0, st>>>(sc, pos, H, scale, talk, L, (__bf16*)hi, (__bf16*)lo);   \
  else talk_softmax_k<float, HM><<<nt, 256, 0, st>>>(sc, pos, H, scale, talk, L, (float*)nullptr, (float*)nullptr);
  if (H <= 8) { BM_HM(8) }
  else if (H <= 16) { BM_HM(16) }
  else if (H <= 32) { BM_HM(32) }
  else { BM_HM(64) }
#undef BM_HM
}

}  // namespace bm
}  // namespace illm
