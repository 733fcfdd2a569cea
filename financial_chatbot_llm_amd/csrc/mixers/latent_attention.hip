// Latent (low-rank key/value) attention over a paged latent cache, with a sliding window.
//
// The cache row of a token is [c: R | k_rot: Dr]: the RMS-normed key/value latent and the one
// rotated key part that all heads share.  Attention runs in the latent space ("absorbed" form):
// the caller folds each head's key up-projection into its query, q_lat[h] = W_uk[h]^T q_nope[h],
// so the score of head h for key j is (q_lat[h] . c_j + q_rot[h] . k_rot_j) * scale and the output
// is o_lat[h] = sum_j p_j c_j; the caller applies the value up-projection to o_lat.  Keys and values
// of all heads are therefore the same cache rows (one read per key serves every head).
//
//   mx_latent_prep    RMS norm of the latent, rotary embedding (interleaved pairs, angle = pos *
//                     inv_freq[i] in f32) of k_rot and of every head's q_rot, cache write.
//   mx_latent_attend  windowed causal softmax attention: query at position p sees keys j with
//                     0 <= p - j < window.  Scores, softmax and accumulation in f32.  The head's
//                     output is multiplied by sigmoid(gate[t, h]) when a gate is given.
#include <stdlib.h>

#include "mx_common.h"

namespace {

constexpr int PAGE = 64;            // tokens per cache page

// one block per token
template <typename T>
__global__ void latent_prep_kernel(const T* __restrict__ kv, long skv, const float* __restrict__ norm_w, float eps,
                                   const float* __restrict__ inv_freq, int rot_dims, const int* __restrict__ pos,
                                   const int* __restrict__ slots, T* __restrict__ cache, const T* __restrict__ q,
                                   long sq, int q_head_stride, int q_rot_off, T* __restrict__ q_rot, int H, int R,
                                   int Dr) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const int slot = slots[t];
  const float p = (float)pos[t];
  const T* row = kv + t * skv;
  const int D = R + Dr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = ldf(row + i);
    ss += v * v;
  }
  ss = mx_block_sum(ss, scratch);
  const float k = 1.0f / sqrtf(ss / (float)R + eps);
  if (slot >= 0) {
    T* dst = cache + (long)slot * D;
    for (int i = threadIdx.x; i < R; i += blockDim.x) stf(dst + i, ldf(row + i) * k * norm_w[i]);
    for (int i = threadIdx.x; i < Dr / 2; i += blockDim.x) {
      const float u = ldf(row + R + 2 * i), v = ldf(row + R + 2 * i + 1);
      if (2 * i + 1 < rot_dims) {
        float sn, cs;
        sincosf(p * inv_freq[i], &sn, &cs);
        stf(dst + R + 2 * i, u * cs - v * sn);
        stf(dst + R + 2 * i + 1, v * cs + u * sn);
      } else {
        stf(dst + R + 2 * i, u);
        stf(dst + R + 2 * i + 1, v);
      }
    }
    if ((Dr & 1) && threadIdx.x == 0) stf(dst + R + Dr - 1, ldf(row + R + Dr - 1));
  }
  // queries: head h's rotated part is q[t][h * q_head_stride + q_rot_off ..+Dr]
  const int half = Dr / 2;
  for (int e = threadIdx.x; e < H * half; e += blockDim.x) {
    const int h = e / half, i = e - h * half;
    const T* qs = q + t * sq + (long)h * q_head_stride + q_rot_off;
    T* qd = q_rot + (t * H + h) * Dr;
    const float u = ldf(qs + 2 * i), v = ldf(qs + 2 * i + 1);
    if (2 * i + 1 < rot_dims) {
      float sn, cs;
      sincosf(p * inv_freq[i], &sn, &cs);
      stf(qd + 2 * i, u * cs - v * sn);
      stf(qd + 2 * i + 1, v * cs + u * sn);
    } else {
      stf(qd + 2 * i, u);
      stf(qd + 2 * i + 1, v);
    }
  }
  if (Dr & 1)
    for (int h = threadIdx.x; h < H; h += blockDim.x)
      stf(q_rot + (t * H + h) * Dr + Dr - 1, ldf(q + t * sq + (long)h * q_head_stride + q_rot_off + Dr - 1));
}

// Work layout: a block owns QT consecutive rows of one segment and HB heads; its QT*HB (row, head)
// items are dealt round-robin to the 4 waves (<= ITEMS per wave).  Key tiles of KT cache rows are
// staged in LDS once per block and shared by all items.  Per item and tile:
//   phase 1  lane j scores key j (q read from a per-wave LDS copy: broadcast; the key row stride
//            is odd in 4-byte words: conflict-free),
//   phase 2  lane l accumulates value columns l, l+64, ... over the tile's keys.
constexpr int ATT_WAVES = 4;
constexpr int ATT_ITEMS = 8;        // items per wave
constexpr int ATT_RPL = 8;          // value columns per lane: R <= 512

template <typename T>
__global__ void __launch_bounds__(ATT_WAVES * 64)
latent_attend_kernel(const T* __restrict__ q_lat, const T* __restrict__ q_rot, const T* __restrict__ cache,
                     const int* __restrict__ cu, const int* __restrict__ pos, const int* __restrict__ bt, int btw,
                     const T* __restrict__ gate, long sgate, int window, float scale, T* __restrict__ out,
                     int H, int R, int Dr, int QT, int HB, int KT, int ldk) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int D = R + Dr;
  T* ktile = reinterpret_cast<T*>(smem);                                  // [KT][ldk]
  float* qbuf = reinterpret_cast<float*>(smem + (((size_t)KT * ldk * sizeof(T) + 15) & ~(size_t)15));  // [4][D]
  float* pbuf = qbuf + ATT_WAVES * D;                                     // [4][64]
  const int s = blockIdx.z;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  const int t0 = blockIdx.x * QT;
  if (t0 >= n) return;
  const int nq = min(QT, n - t0);
  const int h0 = blockIdx.y * HB;
  const int nh = min(HB, H - h0);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int p_first = pos[r0 + t0], p_last = pos[r0 + t0 + nq - 1];
  const int lo = max(0, p_first - window + 1);
  const int nitems = nq * nh;
  float* myq = qbuf + wave * D;
  float* myp = pbuf + wave * 64;

  float m[ATT_ITEMS], l[ATT_ITEMS], acc[ATT_ITEMS][ATT_RPL];
#pragma unroll
  for (int i = 0; i < ATT_ITEMS; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
#pragma unroll
    for (int c = 0; c < ATT_RPL; ++c) acc[i][c] = 0.f;
  }

  for (int k0 = (lo / KT) * KT; k0 <= p_last; k0 += KT) {
    __syncthreads();                       // previous tile fully consumed
    const int rows = min(KT, p_last + 1 - k0);   // only these rows of the tile are staged (and read)
    {
      const long base = ((long)bt[(long)s * btw + k0 / PAGE] * PAGE + (k0 % PAGE)) * D;
      for (int e = threadIdx.x; e < rows * D; e += blockDim.x) {
        const int j = e / D, d = e - j * D;
        ktile[j * ldk + d] = cache[base + e];
      }
    }
    __syncthreads();
#pragma unroll
    for (int ii = 0; ii < ATT_ITEMS; ++ii) {
      const int item = wave + ii * ATT_WAVES;
      if (item >= nitems) continue;                       // wave-uniform
      const int tq = item / nh, hh = item - tq * nh;
      const long row = r0 + t0 + tq;
      const int h = h0 + hh;
      const int p = pos[row];
      const int j = k0 + lane;
      const bool vis = lane < rows && j <= p && j > p - window;
      if (__ballot(vis) == 0ull) continue;                // no visible key of this tile
      // this item's query into the wave's LDS copy
      {
        const T* ql = q_lat + (row * H + h) * R;
        const T* qr = q_rot + (row * H + h) * Dr;
        for (int d = lane; d < D; d += 64) myq[d] = d < R ? ldf(ql + d) : ldf(qr + d - R);
      }
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
      for (int c = 0; c < ATT_RPL; ++c) {
        const int d = lane + 64 * c;
        if (d < R) {
          float a = acc[ii][c] * corr;
          for (int jj = 0; jj < rows; ++jj) a += myp[jj] * ldf(ktile + jj * ldk + d);
          acc[ii][c] = a;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
#pragma unroll
  for (int ii = 0; ii < ATT_ITEMS; ++ii) {
    const int item = wave + ii * ATT_WAVES;
    if (item >= nitems) continue;
    const int tq = item / nh, hh = item - tq * nh;
    const long row = r0 + t0 + tq;
    const int h = h0 + hh;
    float g = 1.0f / l[ii];
    if (gate != nullptr) g *= mx_sigmoid(ldf(gate + row * sgate + h));
#pragma unroll
    for (int c = 0; c < ATT_RPL; ++c) {
      const int d = lane + 64 * c;
      if (d < R) stf(out + (row * H + h) * R + d, acc[ii][c] * g);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// bf16 on the matrix cores (v_mfma_f32_16x16x32_bf16).  A block owns 64 (row, head) pairs of one
// segment -- QT consecutive rows x HB heads, 16 pairs per wave -- and walks the key tiles of the
// union of their windows, KT = 32 keys at a time.  Per tile and wave:
//     S^T = K . Q^T      A: key rows from LDS (16-byte reads), B: the wave's queries, in registers
//     online softmax     the statistics of query (lane % 16) live in that lane, f32
//     O^T += V^T . P^T   A: the latent part of the tile, transposed in LDS; B: P straight from the
//                        S^T registers (the MFMA's k slots 8g+i / 8g+4+i hold keys 4g+i / 16+4g+i)
// Feature dimensions are zero-padded to multiples of 32 (keys) / 16 (values) in LDS and registers.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int MKT = 32;             // keys per tile
constexpr int MLDV = MKT + 8;       // row stride of the transposed value tile

template <int KSM, int NTM>         // up to 32*KSM key dims, 16*NTM value dims
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))   // two blocks per CU: <= 256 registers
latent_attend_mfma_kernel(const bf16* __restrict__ q_lat, const bf16* __restrict__ q_rot,
                          const bf16* __restrict__ cache, const int* __restrict__ cu, const int* __restrict__ pos,
                          const int* __restrict__ bt, int btw, const bf16* __restrict__ gate, long sgate, int window,
                          float scale, bf16* __restrict__ out, int H, int R, int Dr, int QT, int HB, int nsplit,
                          float* __restrict__ ws) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int D = R + Dr;
  const int KS = (D + 31) / 32, NT = (R + 15) / 16;
  const int ldk = KS * 32 + 8;
  bf16* kt_lds = reinterpret_cast<bf16*>(smem);                 // [MKT][ldk]
  bf16* vt_lds = kt_lds + MKT * ldk;                            // [NT*16][MLDV]
  const int s = blockIdx.z;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  // nsplit > 1 (single-row segments): blockIdx.x is the part of the key range this block walks
  const int split = nsplit > 1 ? blockIdx.x : 0;
  const int t0 = nsplit > 1 ? 0 : blockIdx.x * QT;
  if (t0 >= n) return;
  const int nq = min(QT, n - t0);
  const int h0 = blockIdx.y * HB;
  const int nh = min(HB, H - h0);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;
  const int p_first = pos[r0 + t0], p_last = pos[r0 + t0 + nq - 1];
  const int lo = max(0, p_first - window + 1);
  // this lane's query: pair index 16 * wave + c
  const int pair = 16 * wave + c;
  const bool qok = pair < nq * nh;
  const int tq = qok ? pair / nh : 0, hh = qok ? pair - (pair / nh) * nh : 0;
  const long row = r0 + t0 + tq;
  const int h = h0 + hh;
  const int pq = qok ? pos[row] : -1;
  const bool wave_live = 16 * wave < nq * nh;

  bf16x8 qf[KSM];
#pragma unroll
  for (int ks = 0; ks < KSM; ++ks) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = 32 * ks + 8 * g + e;
      float v = 0.f;
      if (qok && d < D) v = d < R ? (float)q_lat[(row * H + h) * R + d] : (float)q_rot[(row * H + h) * Dr + d - R];
      qf[ks][e] = (bf16)v;
    }
  }
  f32x4 o[NTM];
#pragma unroll
  for (int nt = 0; nt < NTM; ++nt) o[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // zero the padding columns / rows once (staging only writes real elements); nothing to do when the
  // 16-byte staging path covers every column the MFMAs read
  if ((D & 31) != 0 || (R & 15) != 0) {
    unsigned* z = reinterpret_cast<unsigned*>(smem);
    const int words = (MKT * ldk + NT * 16 * MLDV) / 2;
    for (int e = threadIdx.x; e < words; e += 256) z[e] = 0u;
  }

  int k_begin = (lo / MKT) * MKT, k_end = p_last;     // first tile start, last key
  if (nsplit > 1) {
    const int tiles = (p_last - k_begin) / MKT + 1;
    const int per = (tiles + nsplit - 1) / nsplit;
    k_begin += split * per * MKT;
    k_end = min(p_last, k_begin + per * MKT - 1);
  }
  // staging, 16-byte path (rows are whole 16-byte pieces): a work item is a pair of keys x 8 dims --
  // two row loads, two 16-byte stores into the key tile and eight 4-byte stores (one key pair
  // each) into the transposed value tile.  The next tile's loads are issued before the current
  // tile's MFMAs and land in registers while they run.
  constexpr int MAXIT = 3;                   // 16 pairs * (<= 40 pieces) / 256 threads
  const bool v16 = (D & 7) == 0;
  const int d8 = D >> 3;
  bf16x8 pre[MAXIT][2];
  auto load_tile = [&](int k0) {
    const int rows = min(MKT, p_last + 1 - k0);
    const bf16* src = cache + ((long)bt[(long)s * btw + k0 / PAGE] * PAGE + (k0 % PAGE)) * D;
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) {
      const int e = min((int)threadIdx.x + 256 * it, 16 * d8 - 1);
      const int d = (e >> 4) * 8, jp = e & 15;
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int j = 2 * jp + r;
        bf16x8 v = *reinterpret_cast<const bf16x8*>(src + (long)min(j, rows - 1) * D + d);
        if (j >= rows)
#pragma unroll
          for (int i = 0; i < 8; ++i) v[i] = (bf16)0.f;
        pre[it][r] = v;
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) {
      const int e = threadIdx.x + 256 * it;
      if (e < 16 * d8) {
        const int d = (e >> 4) * 8, jp = e & 15;
        *reinterpret_cast<bf16x8*>(kt_lds + (2 * jp) * ldk + d) = pre[it][0];
        *reinterpret_cast<bf16x8*>(kt_lds + (2 * jp + 1) * ldk + d) = pre[it][1];
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (d + i < R) {
            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
            *reinterpret_cast<bf16x2*>(vt_lds + (d + i) * MLDV + 2 * jp) = bf16x2{pre[it][0][i], pre[it][1][i]};
          }
      }
    }
  };
  if (v16 && k_begin <= k_end) load_tile(k_begin);
  for (int k0 = k_begin; k0 <= k_end; k0 += MKT) {
    __syncthreads();
    const int rows = min(MKT, p_last + 1 - k0);
    if (v16) {
      store_tile();
    } else {
      const long base = ((long)bt[(long)s * btw + k0 / PAGE] * PAGE + (k0 % PAGE)) * D;
      for (int e = threadIdx.x; e < MKT * D; e += 256) {
        const int j = e / D, d = e - j * D;
        const bf16 v = j < rows ? cache[base + e] : (bf16)0.f;
        kt_lds[j * ldk + d] = v;
        if (d < R) vt_lds[d * MLDV + j] = v;
      }
    }
    __syncthreads();
    if (v16 && k0 + MKT <= k_end) load_tile(k0 + MKT);
    if (!wave_live) continue;
    // S^T for the two 16-key halves
    f32x4 st[2];
    float sc[2][4];
    float tmax = -INFINITY;
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      st[kh] = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16* kr = kt_lds + (16 * kh + c) * ldk + 8 * g;
#pragma unroll
      for (int ks = 0; ks < KSM; ++ks)
        if (ks < KS) st[kh] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(kr + 32 * ks), qf[ks], st[kh], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = k0 + 16 * kh + 4 * g + i;
        const bool vis = j <= pq && j > pq - window;
        sc[kh][i] = vis ? st[kh][i] * scale : -INFINITY;
        tmax = fmaxf(tmax, sc[kh][i]);
      }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float mn = fmaxf(m, tmax);
    const float corr = (m == -INFINITY) ? 0.f : expf(m - mn);
    bf16x8 pb;
    float psum = 0.f;
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = sc[kh][i] == -INFINITY ? 0.f : expf(sc[kh][i] - mn);
        psum += p;
        pb[4 * kh + i] = (bf16)p;
      }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = mn;
#pragma unroll
    for (int nt = 0; nt < NTM; ++nt) {
      if (nt < NT) {
        const bf16* vr = vt_lds + (16 * nt + c) * MLDV + 4 * g;
        const bf16x4 a0 = *reinterpret_cast<const bf16x4*>(vr), a1 = *reinterpret_cast<const bf16x4*>(vr + 16);
        bf16x8 a;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[i] = a0[i];
          a[4 + i] = a1[i];
        }
        o[nt] *= corr;
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, o[nt], 0, 0, 0);
      }
    }
  }
  if (!qok) return;
  if (nsplit > 1) {                          // unnormalised part: o | m | l, merged by latent_merge_kernel
    float* w = ws + ((row * H + h) * nsplit + split) * (long)(R + 2);
#pragma unroll
    for (int nt = 0; nt < NTM; ++nt)
      if (nt < NT)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * nt + 4 * g + i;
          if (r < R) w[r] = o[nt][i];
        }
    if (g == 0) {
      w[R] = m;
      w[R + 1] = l;
    }
    return;
  }
  float gsc = 1.0f / l;
  if (gate != nullptr) gsc *= mx_sigmoid((float)gate[row * sgate + h]);
  bf16* dst = out + (row * H + h) * R;
#pragma unroll
  for (int nt = 0; nt < NTM; ++nt) {
    if (nt < NT) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * nt + 4 * g + i;
        if (r < R) dst[r] = (bf16)(o[nt][i] * gsc);
      }
    }
  }
}

// grid (rows, H): combine the nsplit parts of one (row, head)
__global__ void latent_merge_kernel(const float* __restrict__ ws, const bf16* __restrict__ gate, long sgate,
                                    bf16* __restrict__ out, int H, int R, int nsplit) {
  const long row = blockIdx.x;
  const int h = blockIdx.y;
  const float* w = ws + (row * H + h) * nsplit * (long)(R + 2);
  float M = -INFINITY;
  for (int i = 0; i < nsplit; ++i) M = fmaxf(M, w[i * (R + 2) + R]);
  float L = 0.f;
  for (int i = 0; i < nsplit; ++i) {
    const float mi = w[i * (R + 2) + R];
    if (mi != -INFINITY) L += w[i * (R + 2) + R + 1] * expf(mi - M);
  }
  float gsc = 1.0f / L;
  if (gate != nullptr) gsc *= mx_sigmoid((float)gate[row * sgate + h]);
  for (int r = threadIdx.x; r < R; r += blockDim.x) {
    float a = 0.f;
    for (int i = 0; i < nsplit; ++i) {
      const float mi = w[i * (R + 2) + R];
      if (mi != -INFINITY) a += w[i * (R + 2) + r] * expf(mi - M);
    }
    out[(row * H + h) * R + r] = (bf16)(a * gsc);
  }
}

}  // namespace

// MX_ATTEND_MFMA=0 keeps every call on the f32-lane kernel (A/B and debugging)
static bool mx_use_mfma() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("MX_ATTEND_MFMA");
    v = (e != nullptr && e[0] == '0') ? 0 : 1;
  }
  return v == 1;
}

// kv [T, R+Dr] slice (row stride skv); q [T, ...] with head h's rotated part at h*q_head_stride+q_rot_off
// (row stride sq); q_rot out [T, H, Dr]; cache [pages*64, R+Dr]; all of storage type dt
MX_API int mx_latent_prep(const void* kv, long skv, const float* norm_w, float eps, const float* inv_freq,
                          int rot_dims, const int* pos, const int* slots, void* cache, const void* q, long sq,
                          int q_head_stride, int q_rot_off, void* q_rot, int dt, int T, int H, int R, int Dr,
                          hipStream_t st) {
  if (T <= 0) return 0;
  MX_DISPATCH(dt, TT, latent_prep_kernel<TT><<<T, 256, 0, st>>>((const TT*)kv, skv, norm_w, eps, inv_freq, rot_dims,
                                                                pos, slots, (TT*)cache, (const TT*)q, sq,
                                                                q_head_stride, q_rot_off, (TT*)q_rot, H, R, Dr));
  MX_RETURN_LAUNCH();
}

// q_lat [T, H, R], q_rot [T, H, Dr], out [T, H, R] contiguous; cu [S+1] row bounds of the segments,
// pos [T] positions, bt [S, btw] page tables; gate [T, >=H] slice (row stride sgate) or null.
// nsplit > 1 with a workspace ws (f32 [T, H, nsplit, R + 2]) and single-row segments: the key range of
// each row is walked by nsplit blocks and merged (bf16 matrix-core form only; ignored otherwise).
MX_API int mx_latent_attend(const void* q_lat, const void* q_rot, const void* cache, const int* cu, const int* pos,
                            const int* bt, int btw, const void* gate, long sgate, int window, float scale,
                            void* out, int dt, int S, int max_len, int H, int R, int Dr, int nsplit, float* ws,
                            hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (R > 64 * ATT_RPL) return (int)hipErrorInvalidValue;
  const int D = R + Dr;
  if (dt == 0 && D <= 320 && R <= 256 && mx_use_mfma()) {
    // matrix-core form: 64 (row, head) pairs per block
    const int HB = H < 64 ? H : 64;
    const int QT = max_len == 1 ? 1 : (64 / HB > 0 ? 64 / HB : 1);
    const int KS = (D + 31) / 32, NT = (R + 15) / 16;
    const size_t lds = ((size_t)MKT * (KS * 32 + 8) + (size_t)NT * 16 * MLDV) * sizeof(bf16);
    if (max_len != 1 || ws == nullptr || nsplit < 1) nsplit = 1;
    dim3 grid(nsplit > 1 ? nsplit : (max_len + QT - 1) / QT, (H + HB - 1) / HB, S);
    if (D <= 128 && R <= 128)
      latent_attend_mfma_kernel<4, 8><<<grid, 256, lds, st>>>(
          (const bf16*)q_lat, (const bf16*)q_rot, (const bf16*)cache, cu, pos, bt, btw, (const bf16*)gate, sgate,
          window, scale, (bf16*)out, H, R, Dr, QT, HB, nsplit, ws);
    else
      latent_attend_mfma_kernel<10, 16><<<grid, 256, lds, st>>>(
          (const bf16*)q_lat, (const bf16*)q_rot, (const bf16*)cache, cu, pos, bt, btw, (const bf16*)gate, sgate,
          window, scale, (bf16*)out, H, R, Dr, QT, HB, nsplit, ws);
    if (nsplit > 1) {
      dim3 g2(S, H);           // single-row segments: row index == segment index
      latent_merge_kernel<<<g2, R >= 128 ? 128 : 64, 0, st>>>(ws, (const bf16*)gate, sgate, (bf16*)out, H, R, nsplit);
    }
    MX_RETURN_LAUNCH();
  }
  const int esz = dt == 1 ? 4 : 2;
  // key row stride: odd in 4-byte words
  int ldk = D;
  if (esz == 4) ldk += (ldk & 1) ? 0 : 1;
  else {
    ldk += ldk & 1;
    if (((ldk / 2) & 1) == 0) ldk += 2;
  }
  int KT = 64;
  while (KT > 8 && (size_t)KT * ldk * esz > 40 * 1024) KT >>= 1;
  // decode-like steps (one row per segment): all items are heads; prompt chunks: 4 rows x 8 heads
  const int QT = max_len == 1 ? 1 : 4;
  int HB = (ATT_WAVES * ATT_ITEMS) / QT;
  if (HB > H) HB = H;
  const size_t lds = (((size_t)KT * ldk * esz + 15) & ~(size_t)15) + (size_t)ATT_WAVES * (D + 64) * sizeof(float);
  if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
  dim3 grid((max_len + QT - 1) / QT, (H + HB - 1) / HB, S);
  MX_DISPATCH(dt, TT, latent_attend_kernel<TT><<<grid, ATT_WAVES * 64, lds, st>>>(
      (const TT*)q_lat, (const TT*)q_rot, (const TT*)cache, cu, pos, bt, btw, (const TT*)gate, sgate, window, scale,
      (TT*)out, H, R, Dr, QT, HB, KT, ldk));
  MX_RETURN_LAUNCH();
}
