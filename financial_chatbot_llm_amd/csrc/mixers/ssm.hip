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
#include "mx_common.h"

namespace {

constexpr int CONV_TT = 32;   // tokens per block of the convolution
constexpr int MAX_TAPS = 8;

// grid (ceil(C/256), ceil(max_len/CONV_TT), S)
template <typename T>
__global__ void conv_silu_kernel(const T* __restrict__ in, long si, const float* __restrict__ w,
                                 const float* __restrict__ bias, const float* __restrict__ state,
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
      win[k + 1] = j >= 0 ? ldf(in + (long)(r0 + j) * si + c) : (fresh ? 0.f : st[(long)(K - 1 + j) * C + c]);
    }
  }
  const float b = bias != nullptr ? bias[c] : 0.f;
  const int t1 = min(t0 + CONV_TT, n);
  for (int i = t0; i < t1; ++i) {
#pragma unroll
    for (int k = 0; k < MAX_TAPS - 1; ++k) win[k] = win[k + 1];
    // after the shift the newest input goes to tap K-1
    const float v = ldf(in + (long)(r0 + i) * si + c);
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k) if (k == K - 1) win[k] = v;
    float acc = b;
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k) if (k < K) acc += wk[k] * win[k];
    out[(long)(r0 + i) * C + c] = mx_silu(acc);
  }
}

// grid (ceil(C/256), S): the slot's last K-1 inputs after this chunk.  Runs after conv_silu_kernel
// of the same step (same stream).  One thread owns a channel's K-1 entries and walks them upward,
// reading entry j + n before it writes entry j, so the shift is safe in place.
template <typename T>
__global__ void conv_state_kernel(const T* __restrict__ in, long si, float* __restrict__ state,
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
    if (i >= 0) v = ldf(in + (long)(r0 + i) * si + c);
    else v = fresh ? 0.f : st[(long)(j + n) * C + c];
    st[(long)j * C + c] = v;
  }
}

// Sequential scan.  grid (ceil(P/PT), H, S), block PT * NS threads: thread (p, ns) keeps the state
// entries S[p][ns + NS*i] in registers; the NS partial sums of y_t[p] are reduced inside the wave.
// The rows of a chunk of TB tokens (B_t, C_t, the block's x_t, dt and the decay) are staged in LDS;
// the next chunk's rows are fetched into registers while the current chunk's TB dependent steps
// run, so the recurrence never waits on HBM.
constexpr int SCAN_NS = 16;       // lanes sharing one value channel
constexpr int SCAN_PT = 16;       // value channels per block (256 threads)
constexpr int SCAN_NI = 16;       // state entries per lane: N <= 256
constexpr int SCAN_PF = 36;       // prefetch registers per thread: TB * (2N + PT + 2) <= 256 * SCAN_PF

template <typename TD>
__global__ void __launch_bounds__(SCAN_PT * SCAN_NS)
ssm_scan_kernel(const float* __restrict__ u, int C, const TD* __restrict__ dt_raw, long sdt,
                const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dp,
                float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ slot,
                const int* __restrict__ pos, float* __restrict__ y, int H, int P, int N, int G, int TB) {
  extern __shared__ float rows[];            // [TB][RW]
  const int s = blockIdx.z;
  const int sl = slot[s];
  if (sl < 0) return;
  const int h = blockIdx.y;
  const int ns = threadIdx.x % SCAN_NS;
  const int pl = threadIdx.x / SCAN_NS;
  const int p0 = blockIdx.x * SCAN_PT;
  const int p = p0 + pl;
  const bool live = p < P;
  const int pc = live ? p : P - 1;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  if (n <= 0) return;
  const int g = h / (H / G);
  const bool fresh = pos[r0] == 0;
  const int inner = H * P;
  const int RW = 2 * N + SCAN_PT + 2;
  float* sp = state + (((long)sl * H + h) * P + pc) * N;
  float S[SCAN_NI];
#pragma unroll
  for (int i = 0; i < SCAN_NI; ++i) {
    const int k = ns + SCAN_NS * i;
    S[i] = (!fresh && k < N) ? sp[k] : 0.f;
  }
  const float A = -expf(A_log[h]);
  const float bias = dt_bias[h], Dh = Dp[h];
  float pf[SCAN_PF];

  auto fetch = [&](int c0) {                 // rows c0 .. c0+TB-1 of the segment -> pf
    const int cnt = min(TB, n - c0) * RW;
#pragma unroll
    for (int j = 0; j < SCAN_PF; ++j) {
      const int e = threadIdx.x + j * (SCAN_PT * SCAN_NS);
      float v = 0.f;
      if (e < cnt) {
        const int tt = e / RW, col = e - tt * RW;
        const long r = r0 + c0 + tt;
        const float* ur = u + r * C;
        if (col < N) v = ur[inner + g * N + col];
        else if (col < 2 * N) v = ur[inner + G * N + g * N + (col - N)];
        else if (col < 2 * N + SCAN_PT) {
          const int pp = p0 + col - 2 * N;
          v = pp < P ? ur[h * P + pp] : 0.f;
        } else {
          const float dt = mx_softplus(ldf(dt_raw + r * sdt + h) + bias);
          v = col == 2 * N + SCAN_PT ? dt : expf(A * dt);
        }
      }
      pf[j] = v;
    }
  };

  fetch(0);
  for (int c0 = 0; c0 < n; c0 += TB) {
    const int m = min(TB, n - c0);
    __syncthreads();                         // the previous chunk's readers are done
#pragma unroll
    for (int j = 0; j < SCAN_PF; ++j) {
      const int e = threadIdx.x + j * (SCAN_PT * SCAN_NS);
      if (e < m * RW) rows[e] = pf[j];
    }
    __syncthreads();
    if (c0 + TB < n) fetch(c0 + TB);
    for (int t = 0; t < m; ++t) {
      const float* row = rows + t * RW;
      const float x = row[2 * N + pl];
      const float dt = row[2 * N + SCAN_PT], a = row[2 * N + SCAN_PT + 1];
      const float dx = dt * x;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < SCAN_NI; ++i) {
        const int k = ns + SCAN_NS * i;
        if (k < N) {
          S[i] = a * S[i] + dx * row[k];
          acc += S[i] * row[N + k];
        }
      }
#pragma unroll
      for (int o = SCAN_NS / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
      if (ns == 0 && live) y[(long)(r0 + c0 + t) * inner + h * P + p] = acc + Dh * x;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < SCAN_NI; ++i) {
      const int k = ns + SCAN_NS * i;
      if (k < N) sp[k] = S[i];
    }
  }
}

}  // namespace

// in: [rows, C] slice (row stride si) of the in-projection; out: f32 [rows, C]; state f32 [slots, K-1, C]
MX_API int mx_conv_silu(const void* in, long si, int dt, const float* w, const float* bias, float* state,
                        const int* cu, const int* slot, const int* pos, float* out, int S, int max_len, int C, int K,
                        hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (K < 1 || K > MAX_TAPS) return (int)hipErrorInvalidValue;
  dim3 grid((C + 255) / 256, (max_len + CONV_TT - 1) / CONV_TT, S);
  MX_DISPATCH(dt, TT, conv_silu_kernel<TT><<<grid, 256, 0, st>>>((const TT*)in, si, w, bias, state, cu, slot, pos,
                                                                 out, C, K));
  if (K > 1) {
    dim3 g2((C + 255) / 256, S);
    MX_DISPATCH(dt, TT, conv_state_kernel<TT><<<g2, 256, 0, st>>>((const TT*)in, si, state, cu, slot, pos, C, K));
  }
  MX_RETURN_LAUNCH();
}

// u f32 [rows, C = H*P + 2*G*N]; dt_raw [rows, H] slice (stride sdt, type dt_code); state f32
// [slots, H, P, N]; y f32 [rows, H*P]
MX_API int mx_ssm_scan(const float* u, int C, const void* dt_raw, long sdt, int dt_code, const float* dt_bias,
                       const float* A_log, const float* D, float* state, const int* cu, const int* slot,
                       const int* pos, float* y, int S, int H, int P, int N, int G, hipStream_t st) {
  if (S <= 0) return 0;
  if (N > SCAN_NS * SCAN_NI || G < 1 || H % G) return (int)hipErrorInvalidValue;
  dim3 grid((P + SCAN_PT - 1) / SCAN_PT, H, S);
  const int RW = 2 * N + SCAN_PT + 2;
  int TB = (SCAN_PT * SCAN_NS * SCAN_PF) / RW;
  TB = TB > 32 ? 32 : TB;
  if (TB < 1) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)TB * RW * sizeof(float);
  MX_DISPATCH(dt_code, TT, ssm_scan_kernel<TT><<<grid, SCAN_PT * SCAN_NS, lds, st>>>(
      u, C, (const TT*)dt_raw, sdt, dt_bias, A_log, D, state, cu, slot, pos, y, H, P, N, G, TB));
  MX_RETURN_LAUNCH();
}
