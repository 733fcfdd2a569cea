// State-space (Mamba-2 form) mixer kernels over a flat batch of segments.
//
// A step's rows are `S` segments (a prompt chunk or one decoded token each): segment s owns rows
// cu[s] .. cu[s+1]-1, continues the sequence at position pos[cu[s]] and keeps its recurrent state
// in slot slot[s] (< 0: a padding row, skipped).  A segment that starts at position 0 starts from
// a zero state whatever its slot held before, so a slot needs no clearing when it is handed on.
//
//   conv:  u_t[c] = silu(b[c] + sum_k w[c][k] * in_{t-(K-1)+k}[c]),  inputs before the sequence are 0,
//          inputs before the chunk come from the slot's last K-1 inputs.
//   scan:  per head h (group g = h / (H / G)), state S [P][N] in f32:
//            dt = softplus(dt_raw + dt_bias[h]);  a = exp(-exp(A_log[h]) * dt)
//            S <- a * S + dt * x_t (outer) B_t;   y_t = S C_t + D[h] * x_t
//          u rows are laid out [x: H*P | B: G*N | C: G*N].
#include <type_traits>

#include "mx_common.h"

namespace {

constexpr int CONV_TT = 32;   // tokens per block of the convolution
constexpr int MAX_TAPS = 8;

// grid (ceil(C/256), ceil(max_len/CONV_TT), S)
template <typename T>
__global__ void conv_silu_kernel(const T* __restrict__ in, long si, const float* __restrict__ w,
                                 const float* __restrict__ bias, const float* __restrict__ in_bias, int act,
                                 const float* __restrict__ state,
                                 const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ pos,
                                 float* __restrict__ out, int C, int K) {
  const int s = blockIdx.z;
  const int sl = slot[s];
  if (sl < 0) return;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  const int t0 = blockIdx.y * CONV_TT;
  if (t0 >= n) return;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const bool fresh = pos[r0] == 0;
  const float* st = state + (long)sl * (K - 1) * C;
  float wk[MAX_TAPS], win[MAX_TAPS];
  const float ib = in_bias != nullptr ? in_bias[c] : 0.f;   // added to every real input (the history holds biased inputs)
#pragma unroll
  for (int k = 0; k < MAX_TAPS; ++k) {
    wk[k] = k < K ? w[(long)c * K + k] : 0.f;
    win[k] = 0.f;
  }
  // win[k] holds the input at local index i - (K-1) + k for the current i
#pragma unroll
  for (int k = 0; k < MAX_TAPS - 1; ++k) {
    if (k < K - 1) {
      const int j = t0 - (K - 1) + k;          // local index, may be < 0
      win[k + 1] = j >= 0 ? ldf(in + (long)(r0 + j) * si + c) + ib : (fresh ? 0.f : st[(long)(K - 1 + j) * C + c]);
    }
  }
  const float b = bias != nullptr ? bias[c] : 0.f;
  const int t1 = min(t0 + CONV_TT, n);
  for (int i = t0; i < t1; ++i) {
#pragma unroll
    for (int k = 0; k < MAX_TAPS - 1; ++k) win[k] = win[k + 1];
    // after the shift the newest input goes to tap K-1
    const float v = ldf(in + (long)(r0 + i) * si + c) + ib;
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k) if (k == K - 1) win[k] = v;
    float acc = b;
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k) if (k < K) acc += wk[k] * win[k];
    out[(long)(r0 + i) * C + c] = act == 1 ? mx_silu(acc) : acc;
  }
}

// grid (ceil(C/256), S): the slot's last K-1 inputs after this chunk.  Runs after conv_silu_kernel
// of the same step (same stream).  One thread owns a channel's K-1 entries and walks them upward,
// reading entry j + n before it writes entry j, so the shift is safe in place.
template <typename T>
__global__ void conv_state_kernel(const T* __restrict__ in, long si, const float* __restrict__ in_bias, float* __restrict__ state,
                                  const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ pos,
                                  int C, int K) {
  const int s = blockIdx.y;
  const int sl = slot[s];
  if (sl < 0) return;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  if (n <= 0) return;
  const bool fresh = pos[r0] == 0;
  float* st = state + (long)sl * (K - 1) * C;
  for (int j = 0; j < K - 1; ++j) {
    const int i = n - (K - 1) + j;             // local index of the input that lands in entry j
    float v;
    if (i >= 0) v = ldf(in + (long)(r0 + i) * si + c) + (in_bias != nullptr ? in_bias[c] : 0.f);
    else v = fresh ? 0.f : st[(long)(j + n) * C + c];
    st[(long)j * C + c] = v;
  }
}

// Sequential scan.  grid (ceil(P/PT), H, S), block PT * NS threads: thread (p, ns) keeps the NI
// consecutive state entries S[p][ns*NI .. ns*NI+NI-1] in registers (a wave's state loads and stores
// are contiguous runs of the slot's [P][N] record); the NS partial sums of y_t[p] are reduced
// inside the 16-lane row with DPP swaps.  N is padded to 16 * NI with zeros (B, C and the state
// entries past N stay 0), so the per-token loop has no bounds checks.  The rows of a chunk of TB
// tokens (B_t | C_t, the block's x_t, dt and the decay) are staged in LDS; the next chunk's rows
// are fetched into registers -- unconditional, clamped loads, issued back to back -- before the
// current chunk's TB dependent steps run, so the recurrence never waits on HBM.
constexpr int SCAN_NS = 16;       // lanes sharing one value channel
constexpr int SCAN_PT = 16;       // value channels per block (256 threads)
constexpr int SCAN_PF = 36;       // prefetch registers per thread: TB * 2N <= 256 * SCAN_PF
constexpr int SCAN_NT = SCAN_PT * SCAN_NS;

// sum over the 16 lanes of a DPP row, result in every lane: xor 1, xor 2 (quad permutes), then the
// mirrored 8-lane and 16-lane halves
__device__ __forceinline__ float row_sum16(float v) {
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));   // row_mirror
  return v;
}

// VEC: B | C rows are fetched and staged as 16-byte pieces (N, H*P and the row stride multiples of 4)
template <typename TD, int NI, bool VEC>
__global__ void __launch_bounds__(SCAN_NT) __attribute__((amdgpu_waves_per_eu(NI <= 8 ? 3 : 2)))   // blocks per CU that hide the step latency
ssm_scan_kernel(const float* __restrict__ u, int C, const TD* __restrict__ dt_raw, long sdt,
                const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dp,
                float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ slot,
                const int* __restrict__ pos, float* __restrict__ y, int H, int P, int N, int G, int TB) {
  extern __shared__ __align__(16) float rows[];   // [TB][RW]: B[NP] | C[NP] | x[PT] | dt | decay | pad
  constexpr int NP = SCAN_NS * NI;                // padded state size
  constexpr int RW = 2 * NP + SCAN_PT + 4;
  const int s = blockIdx.z;
  const int sl = slot[s];
  if (sl < 0) return;
  const int h = blockIdx.y;
  const int tid = threadIdx.x;
  const int ns = tid % SCAN_NS;
  const int pl = tid / SCAN_NS;
  const int p0 = blockIdx.x * SCAN_PT;
  const int p = p0 + pl;
  const bool live = p < P;
  const int pc = live ? p : P - 1;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  if (n <= 0) return;
  const int g = h / (H / G);
  const bool fresh = pos[r0] == 0;
  const int inner = H * P;
  const int W2 = 2 * N;
  const int kb = ns * NI;                    // this lane's first state entry
  const bool vec = (NI % 4 == 0) && N == NP; // 16-byte state and LDS accesses
  float* sp = state + (((long)sl * H + h) * P + pc) * N;
  float S[NI];
  if (vec) {
#pragma unroll
    for (int i = 0; i < NI; i += 4) {
      const float4 v = fresh ? float4{0.f, 0.f, 0.f, 0.f} : *reinterpret_cast<const float4*>(sp + kb + i);
      S[i] = v.x;
      S[i + 1 < NI ? i + 1 : i] = v.y;
      S[i + 2 < NI ? i + 2 : i] = v.z;
      S[i + 3 < NI ? i + 3 : i] = v.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < NI; ++i) S[i] = (!fresh && kb + i < N) ? sp[kb + i] : 0.f;
  }
  const float A = -expf(A_log[h]);
  const float bias = dt_bias[h], Dh = Dp[h];
  // B_t | C_t of group g are 2N floats that are contiguous when G == 1, two runs otherwise
  const float* ub = u + inner + g * N;
  const long c_off = (long)(G - 1) * N;      // extra offset of the C run (col >= N)
  // per-thread walk over the chunk's TB x 2N elements (in pieces of UW floats) without divisions
  using U = std::conditional_t<VEC, float4, float>;
  constexpr int UW = VEC ? 4 : 1, PFN = SCAN_PF / UW;
  const int W2u = W2 / UW;
  const int step_t = SCAN_NT / W2u, step_c = SCAN_NT % W2u;
  const int tt0 = tid / W2u, col0 = tid % W2u;
  U pf[PFN];
  float pfx[2], pfd = 0.f;

  // (32-bit element offsets from the block-uniform bases: the launcher checks rows * C < 2^31)
  auto fetch = [&](int c0) {                 // rows c0 .. c0+TB-1 of the segment -> registers
    const int last = n - 1 - c0;             // rows past the segment re-read its last row (never used)
    int tt = tt0, col = col0;
#pragma unroll
    for (int j = 0; j < PFN; ++j) {
      const int r = r0 + c0 + min(tt, last);
      const int ce = col * UW;
      pf[j] = *reinterpret_cast<const U*>(ub + (unsigned)(r * C + ce + (ce >= N ? (int)c_off : 0)));
      col += step_c;
      tt += step_t;
      if (col >= W2u) {
        col -= W2u;
        ++tt;
      }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = tid + j * SCAN_NT;       // (token, channel) of the block's x
      const int tx = e / SCAN_PT, px = p0 + e % SCAN_PT;
      pfx[j] = u[(unsigned)((r0 + c0 + min(tx, last)) * C + h * P + min(px, P - 1))];
    }
    pfd = ldf(dt_raw + (r0 + c0 + min(tid, last)) * sdt + h);
  };

  if (n == 1) {
    // a decoded token: no staging -- every lane reads its own B / C entries and the row's scalars
    const float* ur = u + (long)r0 * C;
    const float dt = mx_softplus(ldf(dt_raw + (long)r0 * sdt + h) + bias);
    const float a = expf(A * dt);
    const float x = ur[h * P + pc];
    const float dx = dt * x;
    const float* Br = ub + (long)r0 * C + kb;
    const float* Cr = Br + N + c_off;
    float acc0 = 0.f, acc1 = 0.f;
    if (vec && (inner & 3) == 0 && (C & 3) == 0) {      // the row's B / C runs are 16-byte aligned too
#pragma unroll
      for (int i = 0; i < NI; i += 4) {
        const float4 b4 = *reinterpret_cast<const float4*>(Br + i), c4 = *reinterpret_cast<const float4*>(Cr + i);
        const float bb[4] = {b4.x, b4.y, b4.z, b4.w}, cc[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int k = i + j < NI ? i + j : i;
          S[k] = a * S[k] + dx * bb[j];
          if (j & 1) acc1 += S[k] * cc[j]; else acc0 += S[k] * cc[j];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NI; ++i)
        if (kb + i < N) {
          S[i] = a * S[i] + dx * Br[i];
          acc0 += S[i] * Cr[i];
        }
    }
    const float acc = row_sum16(acc0 + acc1);
    if (live) {
      if (ns == 0) y[(long)r0 * inner + h * P + p] = acc + Dh * x;
      if (vec) {
#pragma unroll
        for (int i = 0; i < NI; i += 4)
          *reinterpret_cast<float4*>(sp + kb + i) =
              float4{S[i], S[i + 1 < NI ? i + 1 : i], S[i + 2 < NI ? i + 2 : i], S[i + 3 < NI ? i + 3 : i]};
      } else {
#pragma unroll
        for (int i = 0; i < NI; ++i)
          if (kb + i < N) sp[kb + i] = S[i];
      }
    }
    return;
  }
  if (N != NP)                               // the padding columns of B and C stay zero
    for (int e = tid; e < TB * RW; e += SCAN_NT) rows[e] = 0.f;
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += TB) {
    const int m = min(TB, n - c0);
    __syncthreads();                         // the previous chunk's readers are done
    {
      int tt = tt0, col = col0;
#pragma unroll
      for (int j = 0; j < PFN; ++j) {
        const int ce = col * UW;
        if (tt < TB) *reinterpret_cast<U*>(rows + tt * RW + (ce >= N ? ce - N + NP : ce)) = pf[j];
        col += step_c;
        tt += step_t;
        if (col >= W2u) {
          col -= W2u;
          ++tt;
        }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int e = tid + j * SCAN_NT;
        if (e / SCAN_PT < TB) rows[(e / SCAN_PT) * RW + 2 * NP + e % SCAN_PT] = pfx[j];
      }
      if (tid < TB) {
        const float dt = mx_softplus(pfd + bias);
        rows[tid * RW + 2 * NP + SCAN_PT] = dt;
        rows[tid * RW + 2 * NP + SCAN_PT + 1] = expf(A * dt);
      }
    }
    __syncthreads();
    if (c0 + TB < n) fetch(c0 + TB);
    for (int t = 0; t < m; ++t) {
      const float* row = rows + t * RW;
      const float x = row[2 * NP + pl];
      const float2 da = *reinterpret_cast<const float2*>(row + 2 * NP + SCAN_PT);
      const float dx = da.x * x;
      float Bv[NI], Cv[NI];
      if (NI % 4 == 0) {
#pragma unroll
        for (int i = 0; i < NI; i += 4) {
          const float4 b4 = *reinterpret_cast<const float4*>(row + kb + i);
          const float4 c4 = *reinterpret_cast<const float4*>(row + NP + kb + i);
          Bv[i] = b4.x; Bv[i + 1 < NI ? i + 1 : i] = b4.y; Bv[i + 2 < NI ? i + 2 : i] = b4.z; Bv[i + 3 < NI ? i + 3 : i] = b4.w;
          Cv[i] = c4.x; Cv[i + 1 < NI ? i + 1 : i] = c4.y; Cv[i + 2 < NI ? i + 2 : i] = c4.z; Cv[i + 3 < NI ? i + 3 : i] = c4.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          Bv[i] = row[kb + i];
          Cv[i] = row[NP + kb + i];
        }
      }
      float acc = 0.f, acc1 = 0.f;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        S[i] = da.y * S[i] + dx * Bv[i];
        if (i & 1) acc1 += S[i] * Cv[i]; else acc += S[i] * Cv[i];
      }
      acc = row_sum16(acc + acc1);
      if (ns == 0 && live) y[(long)(r0 + c0 + t) * inner + h * P + p] = acc + Dh * x;
    }
  }
  if (live) {
    if (vec) {
#pragma unroll
      for (int i = 0; i < NI; i += 4)
        *reinterpret_cast<float4*>(sp + kb + i) =
            float4{S[i], S[i + 1 < NI ? i + 1 : i], S[i + 2 < NI ? i + 2 : i], S[i + 3 < NI ? i + 3 : i]};
    } else {
#pragma unroll
      for (int i = 0; i < NI; ++i)
        if (kb + i < N) sp[kb + i] = S[i];
    }
  }
}

}  // namespace

// in: [rows, C] slice (row stride si) of the in-projection; out: f32 [rows, C]; state f32 [slots, K-1, C]
// act: 0 none, 1 SiLU; in_bias (optional, [C]) is added to every input before the convolution
MX_API int mx_conv_act(const void* in, long si, int dt, const float* w, const float* bias, const float* in_bias, int act,
                       float* state, const int* cu, const int* slot, const int* pos, float* out, int S, int max_len,
                       int C, int K, hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (K < 1 || K > MAX_TAPS || act < 0 || act > 1) return (int)hipErrorInvalidValue;
  dim3 grid((C + 255) / 256, (max_len + CONV_TT - 1) / CONV_TT, S);
  MX_DISPATCH(dt, TT, conv_silu_kernel<TT><<<grid, 256, 0, st>>>((const TT*)in, si, w, bias, in_bias, act, state, cu,
                                                                 slot, pos, out, C, K));
  if (K > 1) {
    dim3 g2((C + 255) / 256, S);
    MX_DISPATCH(dt, TT, conv_state_kernel<TT><<<g2, 256, 0, st>>>((const TT*)in, si, in_bias, state, cu, slot, pos, C, K));
  }
  MX_RETURN_LAUNCH();
}

MX_API int mx_conv_silu(const void* in, long si, int dt, const float* w, const float* bias, float* state,
                        const int* cu, const int* slot, const int* pos, float* out, int S, int max_len, int C, int K,
                        hipStream_t st) {
  return mx_conv_act(in, si, dt, w, bias, nullptr, 1, state, cu, slot, pos, out, S, max_len, C, K, st);
}

// u f32 [rows, C = H*P + 2*G*N]; dt_raw [rows, H] slice (stride sdt, type dt_code); state f32
// [slots, H, P, N]; y f32 [rows, H*P]
MX_API int mx_ssm_scan(const float* u, int C, const void* dt_raw, long sdt, int dt_code, const float* dt_bias,
                       const float* A_log, const float* D, float* state, const int* cu, const int* slot,
                       const int* pos, float* y, int S, int H, int P, int N, int G, int cu_rows_bound,
                       hipStream_t st) {
  if (S <= 0) return 0;
  if (N > SCAN_NS * 16 || G < 1 || H % G) return (int)hipErrorInvalidValue;
  if ((long)cu_rows_bound * C >= (1L << 31)) return (int)hipErrorInvalidValue;
  dim3 grid((P + SCAN_PT - 1) / SCAN_PT, H, S);
  int TB = (SCAN_NT * SCAN_PF) / (2 * N);
  TB = TB > 32 ? 32 : TB;
  if (TB < 1) return (int)hipErrorInvalidValue;
  const bool vecu = (N % 4 == 0) && ((H * P) % 4 == 0) && (C % 4 == 0);
  const int need = (N + SCAN_NS - 1) / SCAN_NS;         // state entries per lane, rounded up to 1, 2, 4, 8, 16
#define MX_SCAN(NI)                                                                                          \
  do {                                                                                                       \
    const size_t lds = (size_t)TB * (2 * SCAN_NS * NI + SCAN_PT + 4) * sizeof(float);                        \
    if (vecu)                                                                                                \
      MX_DISPATCH(dt_code, TT, ssm_scan_kernel<TT, NI, true><<<grid, SCAN_NT, lds, st>>>(                    \
          u, C, (const TT*)dt_raw, sdt, dt_bias, A_log, D, state, cu, slot, pos, y, H, P, N, G, TB));       \
    else                                                                                                     \
      MX_DISPATCH(dt_code, TT, ssm_scan_kernel<TT, NI, false><<<grid, SCAN_NT, lds, st>>>(                   \
          u, C, (const TT*)dt_raw, sdt, dt_bias, A_log, D, state, cu, slot, pos, y, H, P, N, G, TB));       \
  } while (0)
  if (need <= 1) MX_SCAN(1);
  else if (need <= 2) MX_SCAN(2);
  else if (need <= 4) MX_SCAN(4);
  else if (need <= 8) MX_SCAN(8);
  else MX_SCAN(16);
#undef MX_SCAN
  MX_RETURN_LAUNCH();
}
