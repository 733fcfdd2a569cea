// Token-by-token f32 recurrences over a flat batch of segments (segment s: rows cu[s]..cu[s+1]-1,
// state slot slot[s] (< 0: padding, skipped), zero state when its first row is at position 0).
//
// mx_matrix_scan: a [D, P] state per head with one decay per head and key channel d (acting on row d):
//     gla:    g = sigmoid(a + a_bias)^(1/tau);              S <- g S + k v^T;            o = S^T q
//     delta:  g = exp(-exp(A_log[h]) softplus(a + a_bias));  S <- g S;  u = b (v - S^T k);
//             S <- S + k u^T;  o = S^T q;    q, k unit vectors per head first, b = sigmoid(beta)
//   and q scaled by D^-1/2 in both.  Column p of S never meets another column, so a lane owns RPL
//   rows of one column in registers and LPC neighbouring lanes share a column (D <= RPL * LPC); the
//   two dot products per token are reduced over those lanes with DPP swaps.  The rows of a chunk of
//   tokens (q, k, the decay, the block's v and b) are staged -- and transformed -- in LDS once per
//   block; the outputs of the chunk leave through LDS as whole runs.
//
// mx_lru_scan: a diagonal recurrence per channel, S <- a S + sqrt(1 - a^2) i u with
//     a = exp(-8 sigmoid(zr + r_bias) softplus(lam)),  i = sigmoid(zi + i_bias),
//   output S * gelu_tanh(y + y_bias).
#include "mx_common.h"

namespace {

template <int LPC>
__device__ __forceinline__ float lane_group_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));      // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));      // quad_perm [2,3,0,1]
  if (LPC >= 8) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  if (LPC >= 16) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));  // row_mirror
  return v;
}

__device__ __forceinline__ float ld_code(const void* p, int code, long i) {
  return code == 1 ? reinterpret_cast<const float*>(p)[i] : (float)reinterpret_cast<const bf16*>(p)[i];
}

// grid (ceil(P / CB), H, S), 256 threads = CB columns x LPC lanes, CB = 256 / LPC
template <typename TQ, int RPL, int LPC, bool DELTA>
__global__ void __launch_bounds__(256)
matrix_scan_kernel(const TQ* __restrict__ q, long sq, const TQ* __restrict__ k, long sk, const TQ* __restrict__ v, long sv,
                   const float* __restrict__ a, long sa, const float* __restrict__ a_bias,
                   const float* __restrict__ A_log, const void* __restrict__ beta, long sbeta, int beta_code,
                   float tau_inv, float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ slot,
                   const int* __restrict__ pos, float* __restrict__ out, int H, int G, int D, int P, int TB) {
  extern __shared__ __align__(16) float lds[];
  constexpr int DP = RPL * LPC;          // padded key size
  constexpr int CB = 256 / LPC;          // columns per block
  float* qs = lds;                       // [TB][DP]
  float* ks = qs + TB * DP;              // [TB][DP]
  float* gs = ks + TB * DP;              // [TB][DP]
  float* vs = gs + TB * DP;              // [TB][CB]
  float* os = vs + TB * CB;              // [TB][CB]
  float* bs = os + TB * CB;              // [TB]
  const int s = blockIdx.z;
  const int sl = slot[s];
  if (sl < 0) return;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  if (n <= 0) return;
  const int h = blockIdx.y, kvh = h / (H / G);
  const int tid = threadIdx.x, part = tid % LPC, cl = tid / LPC;
  const int c0 = blockIdx.x * CB, col = c0 + cl;
  const bool fresh = pos[r0] == 0;
  const float qscale = 1.0f / sqrtf((float)D);
  const float eA = DELTA ? expf(A_log[h]) : 0.f;

  float S[RPL];
  float* srec = state + (((long)sl * H + h) * D) * P;
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int d = part * RPL + i;
    S[i] = (!fresh && d < D && col < P) ? srec[(long)d * P + col] : 0.f;
  }

  for (int t0 = 0; t0 < n; t0 += TB) {
    const int nt = min(TB, n - t0);
    // ---- stage the chunk's rows
    for (int e = tid; e < nt * DP; e += 256) {
      const int t = e / DP, d = e - t * DP;
      const long row = r0 + t0 + t;
      float qv = 0.f, kv = 0.f, g = 1.f;
      if (d < D) {
        qv = ldf(q + row * sq + kvh * D + d);
        kv = ldf(k + row * sk + kvh * D + d);
        const float z = a[row * sa + h * D + d] + a_bias[h * D + d];
        if (DELTA) g = expf(-eA * mx_softplus(z));
        else {
          g = expf(-mx_softplus(-z) * tau_inv);          // sigmoid(z)^(1/tau)
          qv *= qscale;
        }
      }
      qs[e] = qv;
      ks[e] = kv;
      gs[e] = g;
    }
    for (int e = tid; e < nt * CB; e += 256) {
      const int t = e / CB, c = e - t * CB;
      vs[e] = c0 + c < P ? ldf(v + (long)(r0 + t0 + t) * sv + h * P + c0 + c) : 0.f;
    }
    if (DELTA)
      for (int t = tid; t < nt; t += 256) bs[t] = mx_sigmoid(ld_code(beta, beta_code, (long)(r0 + t0 + t) * sbeta + h));
    __syncthreads();
    if (DELTA) {      // q and k become unit vectors: one wave per row
      const int wave = tid >> 6, lane = tid & 63;
      for (int r = wave; r < 2 * nt; r += 4) {
        float* buf = r < nt ? qs + r * DP : ks + (r - nt) * DP;
        float ss = 0.f;
        for (int d = lane; d < DP; d += 64) ss += buf[d] * buf[d];
        ss = mx_wave_sum(ss);
        const float sc = (r < nt ? qscale : 1.0f) / sqrtf(ss + 1e-6f);
        for (int d = lane; d < DP; d += 64) buf[d] *= sc;
      }
      __syncthreads();
    }
    // ---- the recurrence
    for (int t = 0; t < nt; ++t) {
      const float4* kr = reinterpret_cast<const float4*>(ks + t * DP + part * RPL);
      const float4* gr = reinterpret_cast<const float4*>(gs + t * DP + part * RPL);
      const float4* qr = reinterpret_cast<const float4*>(qs + t * DP + part * RPL);
      float u = vs[t * CB + cl];
      float kreg[RPL];
#pragma unroll
      for (int i4 = 0; i4 < RPL / 4; ++i4) {
        const float4 kk = kr[i4];
        kreg[4 * i4] = kk.x; kreg[4 * i4 + 1] = kk.y; kreg[4 * i4 + 2] = kk.z; kreg[4 * i4 + 3] = kk.w;
      }
      if (DELTA) {
        float acc = 0.f;
#pragma unroll
        for (int i4 = 0; i4 < RPL / 4; ++i4) {
          const float4 gg = gr[i4];
          S[4 * i4] *= gg.x; S[4 * i4 + 1] *= gg.y; S[4 * i4 + 2] *= gg.z; S[4 * i4 + 3] *= gg.w;
          acc += S[4 * i4] * kreg[4 * i4] + S[4 * i4 + 1] * kreg[4 * i4 + 1] + S[4 * i4 + 2] * kreg[4 * i4 + 2] +
                 S[4 * i4 + 3] * kreg[4 * i4 + 3];
        }
        acc = lane_group_sum<LPC>(acc);
        u = bs[t] * (u - acc);
      }
      float o = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < RPL / 4; ++i4) {
        const float4 qq = qr[i4];
        if (!DELTA) {
          const float4 gg = gr[i4];
          S[4 * i4] *= gg.x; S[4 * i4 + 1] *= gg.y; S[4 * i4 + 2] *= gg.z; S[4 * i4 + 3] *= gg.w;
        }
        S[4 * i4] += kreg[4 * i4] * u;
        S[4 * i4 + 1] += kreg[4 * i4 + 1] * u;
        S[4 * i4 + 2] += kreg[4 * i4 + 2] * u;
        S[4 * i4 + 3] += kreg[4 * i4 + 3] * u;
        o += S[4 * i4] * qq.x + S[4 * i4 + 1] * qq.y + S[4 * i4 + 2] * qq.z + S[4 * i4 + 3] * qq.w;
      }
      o = lane_group_sum<LPC>(o);
      if (part == 0) os[t * CB + cl] = o;
    }
    __syncthreads();
    for (int e = tid; e < nt * CB; e += 256) {
      const int t = e / CB, c = e - t * CB;
      if (c0 + c < P) out[(long)(r0 + t0 + t) * H * P + h * P + c0 + c] = os[e];
    }
    // the next chunk's staging writes qs/ks/gs/vs/bs only; os is rewritten after the barrier that follows it
  }
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int d = part * RPL + i;
    if (d < D && col < P) srec[(long)d * P + col] = S[i];
  }
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// grid (ceil(R / 64), S), 64 threads: one lane per channel
template <typename TY, typename TO>
__global__ void lru_scan_kernel(const float* __restrict__ u, const float* __restrict__ z, int bsz, long T,
                                const float* __restrict__ r_bias, const float* __restrict__ i_bias,
                                const float* __restrict__ lam, const TY* __restrict__ y, long sy,
                                const float* __restrict__ y_bias, float* __restrict__ state, const int* __restrict__ cu,
                                const int* __restrict__ slot, const int* __restrict__ pos, TO* __restrict__ out, int R) {
  const int s = blockIdx.y;
  const int sl = slot[s];
  if (sl < 0) return;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= R) return;
  const int r0 = cu[s], r1 = cu[s + 1];
  if (r1 <= r0) return;
  const int b = c / bsz, j = c - b * bsz;
  const float* zb = z + (long)b * T * 2 * bsz + j;     // block b's rows: [T][zr: bsz | zi: bsz]
  const float sp = mx_softplus(lam[c]), rb = r_bias[c], ib = i_bias[c];
  const float yb = y_bias != nullptr ? y_bias[c] : 0.f;
  float S = pos[r0] == 0 ? 0.f : state[(long)sl * R + c];
#pragma unroll 4
  for (long t = r0; t < r1; ++t) {
    const float r = mx_sigmoid(zb[t * 2 * bsz] + rb);
    const float i = mx_sigmoid(zb[t * 2 * bsz + bsz] + ib);
    const float la = -8.0f * r * sp;                   // log a
    S = expf(la) * S + sqrtf(-expm1f(2.0f * la)) * i * u[t * R + c];
    stf(out + t * R + c, S * gelu_tanh_f(ldf(y + t * sy + c) + yb));
  }
  state[(long)sl * R + c] = S;
}

template <typename TQ, int RPL, int LPC, bool DELTA>
int launch_matrix_scan(const void* q, long sq, const void* k, long sk, const void* v, long sv, const float* a, long sa,
                       const float* a_bias, const float* A_log, const void* beta, long sbeta, int beta_code,
                       float tau_inv, float* state, const int* cu, const int* slot, const int* pos, float* out, int S,
                       int H, int G, int D, int P, hipStream_t st) {
  constexpr int DP = RPL * LPC, CB = 256 / LPC;
  const int per_tok = (3 * DP + 2 * CB + 1) * (int)sizeof(float);
  int TB = (44 * 1024) / per_tok;
  TB = TB > 16 ? 16 : (TB < 1 ? 1 : TB);
  dim3 grid((P + CB - 1) / CB, H, S);
  matrix_scan_kernel<TQ, RPL, LPC, DELTA><<<grid, 256, (size_t)TB * per_tok, st>>>(
      (const TQ*)q, sq, (const TQ*)k, sk, (const TQ*)v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_code, tau_inv, state,
      cu, slot, pos, out, H, G, D, P, TB);
  MX_RETURN_LAUNCH();
}

template <typename TQ, bool DELTA, typename... Args>
int dispatch_matrix_scan(int D, Args... args) {
  if (D <= 32) return launch_matrix_scan<TQ, 8, 4, DELTA>(args...);
  if (D <= 64) return launch_matrix_scan<TQ, 16, 4, DELTA>(args...);
  if (D <= 128) return launch_matrix_scan<TQ, 32, 4, DELTA>(args...);
  if (D <= 256) return launch_matrix_scan<TQ, 32, 8, DELTA>(args...);
  return launch_matrix_scan<TQ, 32, 16, DELTA>(args...);
}

}  // namespace

// q, k [rows, G*D] and v [rows, H*P] slices of storage type dt (row strides sq, sk, sv); a f32 [rows, H*D]
// slice (row stride sa); a_bias f32 [H*D]; delta != 0: A_log f32 [H], beta [rows, >= H] slice of type
// beta_dt; state f32 [slots, H, D, P]; out f32 [rows, H*P].
MX_API int mx_matrix_scan(const void* q, long sq, const void* k, long sk, const void* v, long sv, int dt, const float* a,
                          long sa, const float* a_bias, const float* A_log, const void* beta, long sbeta, int beta_dt,
                          float tau, int delta, float* state, const int* cu, const int* slot, const int* pos,
                          float* out, int S, int H, int G, int D, int P, hipStream_t st) {
  if (S <= 0) return 0;
  if (D < 1 || D > 512 || G < 1 || H % G || (delta && (A_log == nullptr || beta == nullptr)) || tau <= 0.f)
    return (int)hipErrorInvalidValue;
  const float tau_inv = 1.0f / tau;
  if (delta) {
    if (dt == 1)
      return dispatch_matrix_scan<float, true>(D, q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt,
                                               tau_inv, state, cu, slot, pos, out, S, H, G, D, P, st);
    return dispatch_matrix_scan<bf16, true>(D, q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt, tau_inv,
                                            state, cu, slot, pos, out, S, H, G, D, P, st);
  }
  if (dt == 1)
    return dispatch_matrix_scan<float, false>(D, q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt,
                                              tau_inv, state, cu, slot, pos, out, S, H, G, D, P, st);
  return dispatch_matrix_scan<bf16, false>(D, q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt, tau_inv,
                                           state, cu, slot, pos, out, S, H, G, D, P, st);
}

// u f32 [T, R]; z f32 [blocks, T, 2 * R / blocks]; y [T, >= R] slice (row stride sy, type dt_y); state f32
// [slots, R]; out [T, R] of type dt_out
MX_API int mx_lru_scan(const float* u, const float* z, int blocks, const float* r_bias, const float* i_bias,
                       const float* lam, const void* y, long sy, int dt_y, const float* y_bias, float* state,
                       const int* cu, const int* slot, const int* pos, void* out, int dt_out, int S, int R, int T,
                       hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  if (blocks < 1 || R % blocks) return (int)hipErrorInvalidValue;
  dim3 grid((R + 63) / 64, S);
  MX_DISPATCH(dt_y, TY, MX_DISPATCH(dt_out, TO, lru_scan_kernel<TY, TO><<<grid, 64, 0, st>>>(
      u, z, R / blocks, (long)T, r_bias, i_bias, lam, (const TY*)y, sy, y_bias, state, cu, slot, pos, (TO*)out, R)));
  MX_RETURN_LAUNCH();
}
