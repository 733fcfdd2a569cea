// Sliding-window softmax attention with grouped key/value heads over a paged row cache.
//
// The cache row of a token is [k: G*D | v: G*P] (G key/value heads of key size D and value size P).
// Query head h reads key/value head h / (H / G).  The query at position p sees the keys j of its own
// sequence with 0 <= p - j < window; score = q . k * scale; softmax and accumulation in f32; the
// head's output is multiplied by sigmoid(gate[t, h]) when a gate is given.  No positional rotation.
//
//   mx_qk_norm_write   RMS norm over the WHOLE query projection and over the whole key projection
//                      (all heads at once, plain weights), cache write of [normed k | v].
//   mx_window_attend   the attention, over a flat batch of segments (prompt chunks and single
//                      decoded tokens alike).
#include <stdlib.h>

#include "mx_common.h"

namespace {

constexpr int PAGE = 64;            // tokens per cache page

// one block per token
template <typename T>
__global__ void qk_norm_write_kernel(const T* __restrict__ q, long sq, const T* __restrict__ k, long sk,
                                     const T* __restrict__ v, long sv, const float* __restrict__ qw,
                                     const float* __restrict__ kw, float eps, const int* __restrict__ slots,
                                     T* __restrict__ cache, T* __restrict__ qout, int nq, int nk, int nv) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const T* qr = q + t * sq;
  const T* kr = k + t * sk;
  float sq2 = 0.f, sk2 = 0.f;
  if (qw != nullptr)
    for (int i = threadIdx.x; i < nq; i += blockDim.x) {
      const float x = ldf(qr + i);
      sq2 += x * x;
    }
  if (kw != nullptr)
    for (int i = threadIdx.x; i < nk; i += blockDim.x) {
      const float x = ldf(kr + i);
      sk2 += x * x;
    }
  sq2 = mx_block_sum(sq2, scratch);
  sk2 = mx_block_sum(sk2, scratch);
  const float cq = 1.0f / sqrtf(sq2 / (float)nq + eps), ck = 1.0f / sqrtf(sk2 / (float)nk + eps);
  for (int i = threadIdx.x; i < nq; i += blockDim.x)
    stf(qout + t * nq + i, qw != nullptr ? ldf(qr + i) * cq * qw[i] : ldf(qr + i));
  const int slot = slots[t];
  if (slot < 0) return;
  T* dst = cache + (long)slot * (nk + nv);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) stf(dst + i, kw != nullptr ? ldf(kr + i) * ck * kw[i] : ldf(kr + i));
  const T* vr = v + t * sv;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) dst[nk + i] = vr[i];
}

// Work layout: a block owns QT consecutive rows of one segment and HB query heads of ONE key/value
// head; its QT*HB (row, head) items are dealt round-robin to the 4 waves (<= ITEMS per wave).  Tiles
// of KT keys and values of that key/value head are staged in LDS once per block and shared by all
// items.  Per item and tile:
//   phase 1  lane j scores key j (q read from a per-wave LDS copy: broadcast; the key row stride
//            is odd in 4-byte words: conflict-free),
//   phase 2  lane l accumulates value columns l, l+64, ... over the tile's keys.
constexpr int WA_WAVES = 4;
constexpr int WA_ITEMS = 8;         // items per wave
constexpr int WA_CPL = 8;           // value columns per lane: P <= 512

template <typename T>
__global__ void __launch_bounds__(WA_WAVES * 64)
window_attend_kernel(const T* __restrict__ q, long sq, const T* __restrict__ cache, const int* __restrict__ cu,
                     const int* __restrict__ pos, const int* __restrict__ bt, int btw, const T* __restrict__ gate,
                     long sgate, int window, float scale, T* __restrict__ out, int H, int G, int D, int P, int QT,
                     int HB, int KT, int ldk, int ldv) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* ktile = reinterpret_cast<T*>(smem);                                  // [KT][ldk]
  T* vtile = ktile + (size_t)KT * ldk;                                    // [KT][ldv]
  float* qbuf = reinterpret_cast<float*>(smem + ((((size_t)KT * (ldk + ldv)) * sizeof(T) + 15) & ~(size_t)15));  // [4][D]
  float* pbuf = qbuf + WA_WAVES * D;                                      // [4][64]
  const int rep = H / G;
  const int hblocks = (rep + HB - 1) / HB;
  const int s = blockIdx.z;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  const int t0 = blockIdx.x * QT;
  if (t0 >= n) return;
  const int nq = min(QT, n - t0);
  const int g = blockIdx.y / hblocks;                 // key/value head
  const int hg0 = (blockIdx.y - g * hblocks) * HB;    // first query head inside the group
  const int nh = min(HB, rep - hg0);
  const int h0 = g * rep + hg0;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int p_first = pos[r0 + t0], p_last = pos[r0 + t0 + nq - 1];
  const int lo = max(0, p_first - window + 1);
  const int nitems = nq * nh;
  const int Wr = G * (D + P);
  const int koff = g * D, voff = G * D + g * P;
  float* myq = qbuf + wave * D;
  float* myp = pbuf + wave * 64;

  float m[WA_ITEMS], l[WA_ITEMS], acc[WA_ITEMS][WA_CPL];
#pragma unroll
  for (int i = 0; i < WA_ITEMS; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
#pragma unroll
    for (int c = 0; c < WA_CPL; ++c) acc[i][c] = 0.f;
  }

  for (int k0 = (lo / KT) * KT; k0 <= p_last; k0 += KT) {
    __syncthreads();                       // previous tile fully consumed
    const int rows = min(KT, p_last + 1 - k0);   // only these rows of the tile are staged (and read)
    {
      const T* base = cache + ((long)bt[(long)s * btw + k0 / PAGE] * PAGE + (k0 % PAGE)) * Wr;
      for (int e = threadIdx.x; e < rows * D; e += blockDim.x) {
        const int j = e / D, d = e - j * D;
        ktile[j * ldk + d] = base[(long)j * Wr + koff + d];
      }
      for (int e = threadIdx.x; e < rows * P; e += blockDim.x) {
        const int j = e / P, d = e - j * P;
        vtile[j * ldv + d] = base[(long)j * Wr + voff + d];
      }
    }
    __syncthreads();
#pragma unroll
    for (int ii = 0; ii < WA_ITEMS; ++ii) {
      const int item = wave + ii * WA_WAVES;
      if (item >= nitems) continue;                       // wave-uniform
      const int tq = item / nh, hh = item - tq * nh;
      const long row = r0 + t0 + tq;
      const int h = h0 + hh;
      const int p = pos[row];
      const int j = k0 + lane;
      const bool vis = lane < rows && j <= p && j > p - window;
      if (__ballot(vis) == 0ull) continue;                // no visible key of this tile
      {
        const T* qh = q + row * sq + (long)h * D;
        for (int d = lane; d < D; d += 64) myq[d] = ldf(qh + d);
      }
      __builtin_amdgcn_wave_barrier();
      float sc = -INFINITY;
      if (vis) {
        const T* kr = ktile + lane * ldk;
        float a = 0.f;
        for (int d = 0; d < D; ++d) a += myq[d] * ldf(kr + d);
        sc = a * scale;
      }
      const float mt = mx_wave_max(sc);
      const float mn = fmaxf(m[ii], mt);
      const float corr = expf(m[ii] - mn);                 // exp(-inf) = 0 on the first tile
      const float pj = vis ? expf(sc - mn) : 0.f;
      l[ii] = l[ii] * corr + mx_wave_sum(pj);
      m[ii] = mn;
      myp[lane] = pj;
      // one wave writes and reads myq / myp: its LDS accesses complete in program order
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int c = 0; c < WA_CPL; ++c) {
        const int d = lane + 64 * c;
        if (d < P) {
          float a = acc[ii][c] * corr;
          for (int jj = 0; jj < rows; ++jj) a += myp[jj] * ldf(vtile + jj * ldv + d);
          acc[ii][c] = a;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
#pragma unroll
  for (int ii = 0; ii < WA_ITEMS; ++ii) {
    const int item = wave + ii * WA_WAVES;
    if (item >= nitems) continue;
    const int tq = item / nh, hh = item - tq * nh;
    const long row = r0 + t0 + tq;
    const int h = h0 + hh;
    float gs = 1.0f / l[ii];
    if (gate != nullptr) gs *= mx_sigmoid(ldf(gate + row * sgate + h));
#pragma unroll
    for (int c = 0; c < WA_CPL; ++c) {
      const int d = lane + 64 * c;
      if (d < P) stf(out + (row * H + h) * P + d, acc[ii][c] * gs);
    }
  }
}

}  // namespace

// q [T, nq], k [T, nk], v [T, nv] slices (row strides sq, sk, sv); qw [nq], kw [nk] f32 (null: no norm);
// cache [pages*64, nk + nv]; qout [T, nq] contiguous; all of storage type dt
MX_API int mx_qk_norm_write(const void* q, long sq, const void* k, long sk, const void* v, long sv, const float* qw,
                            const float* kw, float eps, const int* slots, void* cache, void* qout, int dt, int T,
                            int nq, int nk, int nv, hipStream_t st) {
  if (T <= 0) return 0;
  MX_DISPATCH(dt, TT, qk_norm_write_kernel<TT><<<T, 256, 0, st>>>((const TT*)q, sq, (const TT*)k, sk, (const TT*)v, sv, qw,
                                                                  kw, eps, slots, (TT*)cache, (TT*)qout, nq, nk, nv));
  MX_RETURN_LAUNCH();
}

// q [T, H*D] (row stride sq), out [T, H*P] contiguous; cu [S+1] row bounds of the segments, pos [T]
// positions, bt [S, btw] page tables; gate [T, >= H] slice (row stride sgate) or null.
MX_API int mx_window_attend(const void* q, long sq, const void* cache, const int* cu, const int* pos, const int* bt,
                            int btw, const void* gate, long sgate, int window, float scale, void* out, int dt, int S,
                            int max_len, int H, int G, int D, int P, hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (P > 64 * WA_CPL || G < 1 || H % G || window < 1) return (int)hipErrorInvalidValue;
  const int rep = H / G;
  const int esz = dt == 1 ? 4 : 2;
  // key row stride: odd in 4-byte words
  int ldk = D;
  if (esz == 4) ldk += (ldk & 1) ? 0 : 1;
  else {
    ldk += ldk & 1;
    if (((ldk / 2) & 1) == 0) ldk += 2;
  }
  const int ldv = P + (esz == 2 ? (P & 1) : 0);
  int KT = 64;
  while (KT > 8 && (size_t)KT * (ldk + ldv) * esz > 40 * 1024) KT >>= 1;
  // decode-like steps (one row per segment): all items are heads of the group; prompt chunks: the
  // group's heads x as many rows as fit in 32 items
  int HB = rep < WA_WAVES * WA_ITEMS ? rep : WA_WAVES * WA_ITEMS;
  int QT = max_len == 1 ? 1 : (WA_WAVES * WA_ITEMS) / HB;
  if (QT < 1) QT = 1;
  const size_t lds = ((((size_t)KT * (ldk + ldv)) * esz + 15) & ~(size_t)15) + (size_t)WA_WAVES * (D + 64) * sizeof(float);
  if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
  dim3 grid((max_len + QT - 1) / QT, G * ((rep + HB - 1) / HB), S);
  MX_DISPATCH(dt, TT, window_attend_kernel<TT><<<grid, WA_WAVES * 64, lds, st>>>(
      (const TT*)q, sq, (const TT*)cache, cu, pos, bt, btw, (const TT*)gate, sgate, window, scale, (TT*)out, H, G, D, P,
      QT, HB, KT, ldk, ldv));
  MX_RETURN_LAUNCH();
}
