// Token-by-token f32 recurrences over a flat batch of segments (segment s: rows cu[s]..cu[s+1]-1,
// state slot slot[s] (< 0: padding, skipped), zero state when its first row is at position 0).
//
// mx_matrix_scan: a [D, P] state per head with one decay per head and key channel d (acting on row d):
//     gla:    g = sigmoid(a + a_bias)^(1/tau);              S <- g S + k v^T;            o = S^T q
//     delta:  g = exp(-exp(A_log[h]) softplus(a + a_bias));  S <- g S;  u = b (v - S^T k);
//             S <- S + k u^T;  o = S^T q;    q, k unit vectors per head first, b = sigmoid(beta)
//   and q scaled by D^-1/2 in both; or (mx_decay_scan) one FIXED decay per head,
//     fixed:  S <- decay[h] S + act(k) act(v)^T;  o = S^T act(q) * out_scale
//   with the activation (none | SiLU) applied while the rows are staged and no prep launch.  Two launches:
//     prep   one block per token, fully parallel: the decays g (written over `a`), and for the delta
//            rule the unit-norm factors of q and k and sigmoid(beta) (steps of single rows -- decode --
//            skip this launch: the scan's one-token form computes them while it stages the row);
//     scan   column p of S never meets another column, so a lane owns RPL rows of one column in
//            registers and LPC neighbouring lanes share a column (D <= RPL * LPC); the two dot
//            products per token are reduced over those lanes with DPP swaps.  The rows of a chunk
//            of TB tokens (q, k, g, the block's v and b) are staged in LDS once per block; the next
//            chunk's rows are fetched into registers -- clamped loads, issued back to back -- before
//            the current chunk's dependent steps run; the chunk's outputs leave through LDS as
//            whole runs.  Steps with few (segment, head) pairs take the variant with more lanes per
//            column so that the grid still covers the chip.
//
// mx_lru_scan: a diagonal recurrence per channel, S <- a S + sqrt(1 - a^2) i u with
//     a = exp(-8 sigmoid(zr + r_bias) softplus(lam)),  i = sigmoid(zi + i_bias),
//   output S * gelu_tanh(y + y_bias).  Two launches: the gates (a, the input term and the GeLU
//   branch: every transcendental; they replace z and u in place, in f32) elementwise over all rows,
//   then the recurrence itself, where a block of 16 channels walks 256 tokens at a time: each thread
//   scans 16 tokens of one channel from zero, the sixteen partial maps S -> A S + B are folded through
//   LDS, and the outputs are corrected by the true start state.  Steps of single rows (decode) take
//   one fused launch instead.
//
// mx_mingru_scan: the minimal gated recurrent unit, S <- (1 - z) S + z c per channel with gates that read
//   only the current token: z = sigmoid(zp + z_bias), u = xp + x_bias, c = u + 1/2 for u >= 0 and
//   sigmoid(u) below; output S * silu(gp).  The same two launches (a gates pass that leaves 1 - z, z c
//   and the SiLU branch in f32, then the recurrence kernel above) or one fused launch for single rows.
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

// one block per token.  a [T, H*D] -> g in place; delta: aux[t] = [rq, rk per key/value head | b per head]
template <typename TQ, bool DELTA>
__global__ void scan_prep_kernel(const TQ* __restrict__ q, long sq, const TQ* __restrict__ k, long sk,
                                 float* __restrict__ a, long sa, const float* __restrict__ a_bias,
                                 const float* __restrict__ A_log, const void* __restrict__ beta, long sbeta,
                                 int beta_code, float tau_inv, float* __restrict__ aux, int H, int G, int D) {
  const long t = blockIdx.x;
  float* ar = a + t * sa;
  for (int e = threadIdx.x; e < H * D; e += blockDim.x) {
    const float z = ar[e] + a_bias[e];
    ar[e] = DELTA ? expf(-expf(A_log[e / D]) * mx_softplus(z)) : expf(-mx_softplus(-z) * tau_inv);
  }
  if (!DELTA) return;
  float* ax = aux + t * (2 * G + H);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const float qscale = 1.0f / sqrtf((float)D);
  for (int r = wave; r < 2 * G; r += nw) {          // row r: q head r / 2 or k head r / 2
    const TQ* src = (r & 1) ? k + t * sk + (r >> 1) * D : q + t * sq + (r >> 1) * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float x = ldf(src + d);
      ss += x * x;
    }
    ss = mx_wave_sum(ss);
    if (lane == 0) ax[r] = ((r & 1) ? 1.0f : qscale) / sqrtf(ss + 1e-6f);
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) ax[2 * G + h] = mx_sigmoid(ld_code(beta, beta_code, t * sbeta + h));
}

// grid (ceil(P / CB), H, S), 256 threads = CB columns x LPC lanes, CB = 256 / LPC
// MODE 0: gla, 1: delta, 2: fixed decay per head (a_bias = decay [H], tau_inv = the output scale, beta_code =
// activation code | storage code of v << 4; q and k of type TQ, no g / aux / beta)
template <typename TQ, int RPL, int LPC, int MODE, bool ONE>      // ONE: every segment is a single row (decode)
__global__ void __launch_bounds__(256)
matrix_scan_kernel(const TQ* __restrict__ q, long sq, const TQ* __restrict__ k, long sk, const TQ* __restrict__ v, long sv,
                   const float* __restrict__ gdec, long sa, const float* __restrict__ aux, float* __restrict__ state,
                   const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ pos,
                   float* __restrict__ out, int H, int G, int D, int P, const float* __restrict__ a_bias,
                   const float* __restrict__ A_log, const void* __restrict__ beta, long sbeta, int beta_code,
                   float tau_inv) {
  constexpr bool DELTA = MODE == 1, FIXED = MODE == 2;
  constexpr int DP = RPL * LPC;          // padded key size
  constexpr int CB = 256 / LPC;          // columns per block
  constexpr int TB = ONE ? 1 : (DP <= 256 ? 16 : 8);   // tokens per chunk
  constexpr int NE = (TB * DP + 255) / 256;            // staged (token, key channel) elements per thread
  constexpr int NV = (TB * CB + 255) / 256;
  __shared__ __align__(16) float qs[TB * DP];
  __shared__ __align__(16) float ks[TB * DP];
  __shared__ __align__(16) float gs[FIXED ? 4 : TB * DP];
  __shared__ float vs[TB * CB];
  __shared__ float os[TB * CB];
  __shared__ float bs[TB];
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
  const int AW = 2 * G + H;              // aux row width
  const float gfix = FIXED ? a_bias[h] : 1.f;
  const int fact = beta_code & 15, vcode = beta_code >> 4;

  float S[RPL];
  float* srec = state + (((long)sl * H + h) * D) * P;
#pragma unroll
  for (int i = 0; i < RPL; ++i) {
    const int d = part * RPL + i;
    S[i] = (!fresh && d < D && col < P) ? srec[(long)d * P + col] : 0.f;
  }

  // chunk rows in flight: element e = tid + 256 * i is (token e / DP, channel e % DP); loads are clamped
  // to the segment's last row and to channel D - 1, and masked when they land
  float pq[NE], pk[NE], pg[NE], pv[NV], pb = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < NE; ++i) {
      const int e = min(tid + 256 * i, TB * DP - 1);
      const int t = e / DP, d = e - t * DP;
      const long row = r0 + min(t0 + t, n - 1);
      const int dc = min(d, D - 1);
      if (FIXED) {         // raw values: the activation waits until they are stored to LDS, so the loads stay in flight
        pq[i] = ldf(q + row * sq + kvh * D + dc);
        pk[i] = ldf(k + row * sk + kvh * D + dc);
      } else if (ONE) {       // no prep pass ran: the decay from its pre-activation here, the unit norms after staging
        pq[i] = ldf(q + row * sq + kvh * D + dc);
        pk[i] = ldf(k + row * sk + kvh * D + dc);
        const float z = gdec[row * sa + h * D + dc] + a_bias[h * D + dc];
        pg[i] = DELTA ? expf(-expf(A_log[h]) * mx_softplus(z)) : expf(-mx_softplus(-z) * tau_inv);
      } else {
        float rq = DELTA ? aux[row * AW + 2 * kvh] : 1.f, rk = DELTA ? aux[row * AW + 2 * kvh + 1] : 1.f;
        pq[i] = ldf(q + row * sq + kvh * D + dc) * rq;
        pk[i] = ldf(k + row * sk + kvh * D + dc) * rk;
        pg[i] = gdec[row * sa + h * D + dc];
      }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = min(tid + 256 * i, TB * CB - 1);
      const int t = e / CB, c = e - t * CB;
      const long vi = (long)(r0 + min(t0 + t, n - 1)) * sv + h * P + min(c0 + c, P - 1);
      if (FIXED) {
        pv[i] = ld_code(v, vcode, vi);
      } else {
        pv[i] = ldf(v + vi);
      }
    }
    if (DELTA && tid < TB)
      pb = ONE ? mx_sigmoid(ld_code(beta, beta_code, (long)(r0 + min(t0 + tid, n - 1)) * sbeta + h))
               : aux[(long)(r0 + min(t0 + tid, n - 1)) * AW + 2 * G + h];
  };
  fetch(0);
  for (int t0 = 0; t0 < n; t0 += TB) {
    const int nt = min(TB, n - t0);
    __syncthreads();                     // the previous chunk's outputs have left os; its rows are consumed
#pragma unroll
    for (int i = 0; i < NE; ++i) {
      const int e = tid + 256 * i;
      if (e < TB * DP) {
        const bool live = (e % DP) < D;
        if (FIXED && fact == 1) {
          qs[e] = live ? mx_silu(pq[i]) : 0.f;
          ks[e] = live ? mx_silu(pk[i]) : 0.f;
        } else {
          qs[e] = live ? pq[i] : 0.f;
          ks[e] = live ? pk[i] : 0.f;
        }
        if (!FIXED) gs[e] = live ? pg[i] : 1.f;
      }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = tid + 256 * i;
      if (e < TB * CB) vs[e] = (c0 + e % CB) < P ? ((FIXED && fact == 1) ? mx_silu(pv[i]) : pv[i]) : 0.f;
    }
    if (DELTA && tid < TB) bs[tid] = pb;
    __syncthreads();
    if (ONE && DELTA) {                  // q (wave 0) and k (wave 1) become unit vectors
      const int wave = tid >> 6, lane = tid & 63;
      if (wave < 2) {
        float* buf = wave == 0 ? qs : ks;
        float ss = 0.f;
        for (int d = lane; d < DP; d += 64) ss += buf[d] * buf[d];
        ss = mx_wave_sum(ss);
        const float sc = (wave == 0 ? qscale : 1.0f) / sqrtf(ss + 1e-6f);
        for (int d = lane; d < DP; d += 64) buf[d] *= sc;
      }
      __syncthreads();
    }
    if (t0 + TB < n) fetch(t0 + TB);
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
        if (FIXED) {
          S[4 * i4] *= gfix; S[4 * i4 + 1] *= gfix; S[4 * i4 + 2] *= gfix; S[4 * i4 + 3] *= gfix;
        } else if (!DELTA) {
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
      if (part == 0) os[t * CB + cl] = DELTA ? o : o * (FIXED ? tau_inv : qscale);   // delta: the scale is part of q's norm factor
    }
    __syncthreads();
    for (int e = tid; e < nt * CB; e += 256) {
      const int t = e / CB, c = e - t * CB;
      if (c0 + c < P) out[(long)(r0 + t0 + t) * H * P + h * P + c0 + c] = os[e];
    }
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

// elementwise over [T, R]: z[.., zr] <- a, z[.., zi] <- sqrt(1 - a^2) i u, then u <- gelu_tanh(y + y_bias)
// (f32: the branch is rounded once, with the product, not before it)
template <typename TY>
__global__ void lru_gates_kernel(float* __restrict__ u, float* __restrict__ z, int bsz, long T,
                                 const float* __restrict__ r_bias, const float* __restrict__ i_bias,
                                 const float* __restrict__ lam, const TY* __restrict__ y, long sy,
                                 const float* __restrict__ y_bias, int R) {
  const long total = T * R;
  for (long e = blockIdx.x * (long)blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
    const long t = e / R;
    const int c = (int)(e - t * R);
    const int b = c / bsz, j = c - b * bsz;
    float* zp = z + ((long)b * T + t) * 2 * bsz + j;
    const float r = mx_sigmoid(zp[0] + r_bias[c]);
    const float i = mx_sigmoid(zp[bsz] + i_bias[c]);
    const float la = -8.0f * r * mx_softplus(lam[c]);             // log a
    zp[0] = expf(la);
    zp[bsz] = sqrtf(-expm1f(2.0f * la)) * i * u[e];               // 1 - a^2 without cancellation
    u[e] = gelu_tanh_f(ldf(y + t * sy + c) + (y_bias != nullptr ? y_bias[c] : 0.f));
  }
}

constexpr int LRU_CL = 16;      // tokens per thread
constexpr int LRU_NC = 16;      // thread chunks per block iteration
constexpr int LRU_CH = 16;      // channels per block (256 threads: 16 channels x 16 chunks, 256 tokens per iteration)

// grid (ceil(R / LRU_CH), S).  z holds a | input term, gy the GeLU branch (lru_gates_kernel).
template <typename TO>
__global__ void __launch_bounds__(256)
lru_scan_kernel(const float* __restrict__ z, const float* __restrict__ gy, int bsz, long T, float* __restrict__ state,
                const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ pos,
                TO* __restrict__ out, int R) {
  __shared__ float sA[LRU_NC][LRU_CH], sB[LRU_NC][LRU_CH], sS[LRU_CH];
  const int s = blockIdx.y;
  const int sl = slot[s];
  if (sl < 0) return;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  if (n <= 0) return;
  const int ch = threadIdx.x % LRU_CH, j = threadIdx.x / LRU_CH;
  const int c = min((int)blockIdx.x * LRU_CH + ch, R - 1);
  const bool live = (int)blockIdx.x * LRU_CH + ch < R;
  const int b = c / bsz, jj = c - b * bsz;
  const float* zb = z + (long)b * T * 2 * bsz + jj;
  if (j == 0) sS[ch] = pos[r0] == 0 ? 0.f : state[(long)sl * R + c];
  for (int t0 = 0; t0 < n; t0 += LRU_CL * LRU_NC) {
    const int first = t0 + j * LRU_CL;
    const int cnt = max(0, min(LRU_CL, n - first));
    float A[LRU_CL], L[LRU_CL], Gy[LRU_CL];
    if (cnt > 0) {
#pragma unroll
      for (int i = 0; i < LRU_CL; ++i) {          // independent loads, issued together
        const long t = r0 + min(first + i, n - 1);
        A[i] = zb[t * 2 * bsz];
        L[i] = zb[t * 2 * bsz + bsz];
        Gy[i] = gy[t * R + c];
      }
    }
    float Pp = 1.f, Ll = 0.f;
#pragma unroll
    for (int i = 0; i < LRU_CL; ++i) {
      if (i < cnt) {
        Ll = A[i] * Ll + L[i];
        Pp *= A[i];
      }
      L[i] = Ll;      // state after token i from a zero start
      A[i] = Pp;      // product of the decays up to token i
    }
    sA[j][ch] = Pp;
    sB[j][ch] = Ll;
    __syncthreads();
    float S0 = sS[ch];
    for (int k = 0; k < j; ++k) S0 = sA[k][ch] * S0 + sB[k][ch];
#pragma unroll
    for (int i = 0; i < LRU_CL; ++i)
      if (i < cnt && live) stf(out + (long)(r0 + first + i) * R + c, (L[i] + A[i] * S0) * Gy[i]);
    __syncthreads();                             // every thread has read sS and the partial maps
    if (j == LRU_NC - 1) sS[ch] = Pp * S0 + Ll;
    __syncthreads();
  }
  if (j == 0 && live) state[(long)sl * R + c] = sS[ch];
}

// steps of single rows (decode): gates, recurrence and output in one launch, one thread per (row, channel)
template <typename TY, typename TO>
__global__ void lru_step_kernel(const float* __restrict__ u, const float* __restrict__ z, int bsz, long T,
                                const float* __restrict__ r_bias, const float* __restrict__ i_bias,
                                const float* __restrict__ lam, const TY* __restrict__ y, long sy,
                                const float* __restrict__ y_bias, float* __restrict__ state, const int* __restrict__ cu,
                                const int* __restrict__ slot, const int* __restrict__ pos, TO* __restrict__ out, int S,
                                int R) {
  const long total = (long)S * R;
  for (long e = blockIdx.x * (long)blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
    const int s = (int)(e / R), c = (int)(e - (long)s * R);
    const int sl = slot[s];
    const long t = cu[s];
    if (sl < 0 || cu[s + 1] <= t) continue;
    const int b = c / bsz, j = c - b * bsz;
    const float* zp = z + ((long)b * T + t) * 2 * bsz + j;
    const float r = mx_sigmoid(zp[0] + r_bias[c]);
    const float i = mx_sigmoid(zp[bsz] + i_bias[c]);
    const float la = -8.0f * r * mx_softplus(lam[c]);
    const float prev = pos[t] == 0 ? 0.f : state[(long)sl * R + c];
    const float Sn = expf(la) * prev + sqrtf(-expm1f(2.0f * la)) * i * u[t * R + c];
    state[(long)sl * R + c] = Sn;
    stf(out + t * R + c, Sn * gelu_tanh_f(ldf(y + t * sy + c) + (y_bias != nullptr ? y_bias[c] : 0.f)));
  }
}

__device__ __forceinline__ float mingru_candidate(float u) { return u >= 0.f ? u + 0.5f : mx_sigmoid(u); }

// elementwise over [T, R]: ab[t, c] <- 1 - z, ab[t, R + c] <- z * candidate, gy[t, c] <- silu(g), all f32
template <typename TI>
__global__ void mingru_gates_kernel(const TI* __restrict__ zp, long sz, const TI* __restrict__ xp, long sx,
                                    const TI* __restrict__ gp, long sg, const float* __restrict__ z_bias,
                                    const float* __restrict__ x_bias, float* __restrict__ ab, float* __restrict__ gy,
                                    long T, int R) {
  const long total = T * R;
  for (long e = blockIdx.x * (long)blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
    const long t = e / R;
    const int c = (int)(e - t * R);
    const float a = ldf(zp + t * sz + c) + (z_bias != nullptr ? z_bias[c] : 0.f);
    const float u = ldf(xp + t * sx + c) + (x_bias != nullptr ? x_bias[c] : 0.f);
    ab[t * 2 * R + c] = mx_sigmoid(-a);                              // 1 - sigmoid(a) without cancellation
    ab[t * 2 * R + R + c] = mx_sigmoid(a) * mingru_candidate(u);
    gy[e] = mx_silu(ldf(gp + t * sg + c));
  }
}

// steps of single rows (decode): gates, recurrence and output in one launch, one thread per (row, channel)
template <typename TI, typename TO>
__global__ void mingru_step_kernel(const TI* __restrict__ zp, long sz, const TI* __restrict__ xp, long sx,
                                   const TI* __restrict__ gp, long sg, const float* __restrict__ z_bias,
                                   const float* __restrict__ x_bias, float* __restrict__ state,
                                   const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ pos,
                                   TO* __restrict__ out, int S, int R) {
  const long total = (long)S * R;
  for (long e = blockIdx.x * (long)blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
    const int s = (int)(e / R), c = (int)(e - (long)s * R);
    const int sl = slot[s];
    const long t = cu[s];
    if (sl < 0 || cu[s + 1] <= t) continue;
    const float a = ldf(zp + t * sz + c) + (z_bias != nullptr ? z_bias[c] : 0.f);
    const float u = ldf(xp + t * sx + c) + (x_bias != nullptr ? x_bias[c] : 0.f);
    const float prev = pos[t] == 0 ? 0.f : state[(long)sl * R + c];
    const float Sn = mx_sigmoid(-a) * prev + mx_sigmoid(a) * mingru_candidate(u);
    state[(long)sl * R + c] = Sn;
    stf(out + t * R + c, Sn * mx_silu(ldf(gp + t * sg + c)));
  }
}

template <typename TQ, int RPL, int LPC, int DELTA>
int launch_matrix_scan(const void* q, long sq, const void* k, long sk, const void* v, long sv, const float* g, long sa,
                       const float* aux, float* state, const int* cu, const int* slot, const int* pos, float* out, int S,
                       int H, int G, int D, int P, const float* a_bias, const float* A_log, const void* beta, long sbeta,
                       int beta_dt, float tau_inv, bool one, hipStream_t st) {
  constexpr int CB = 256 / LPC;
  dim3 grid((P + CB - 1) / CB, H, S);
  if (one)
    matrix_scan_kernel<TQ, RPL, LPC, DELTA, true><<<grid, 256, 0, st>>>(
        (const TQ*)q, sq, (const TQ*)k, sk, (const TQ*)v, sv, g, sa, aux, state, cu, slot, pos, out, H, G, D, P, a_bias,
        A_log, beta, sbeta, beta_dt, tau_inv);
  else
    matrix_scan_kernel<TQ, RPL, LPC, DELTA, false><<<grid, 256, 0, st>>>(
        (const TQ*)q, sq, (const TQ*)k, sk, (const TQ*)v, sv, g, sa, aux, state, cu, slot, pos, out, H, G, D, P, a_bias,
        A_log, beta, sbeta, beta_dt, tau_inv);
  MX_RETURN_LAUNCH();
}

// the variant with 16 lanes per column when the narrow one would leave most of the chip idle
template <typename TQ, int DELTA, typename... Args>
int dispatch_matrix_scan(int D, bool wide, Args... args) {
  if (D <= 32) return launch_matrix_scan<TQ, 8, 4, DELTA>(args...);
  if (D <= 64) return wide ? launch_matrix_scan<TQ, 4, 16, DELTA>(args...) : launch_matrix_scan<TQ, 16, 4, DELTA>(args...);
  if (D <= 128) return wide ? launch_matrix_scan<TQ, 8, 16, DELTA>(args...) : launch_matrix_scan<TQ, 32, 4, DELTA>(args...);
  if (D <= 256) return wide ? launch_matrix_scan<TQ, 16, 16, DELTA>(args...) : launch_matrix_scan<TQ, 32, 8, DELTA>(args...);
  return launch_matrix_scan<TQ, 32, 16, DELTA>(args...);
}

template <typename TQ, bool DELTA>
int run_matrix_scan(const void* q, long sq, const void* k, long sk, const void* v, long sv, float* a, long sa,
                    const float* a_bias, const float* A_log, const void* beta, long sbeta, int beta_dt, float tau_inv,
                    float* aux, float* state, const int* cu, const int* slot, const int* pos, float* out, int S, int T,
                    int H, int G, int D, int P, int max_len, hipStream_t st) {
  const bool one = max_len == 1;         // every segment is a single row: no chunk staging
  if (!one)        // single-row steps fold this pass into the scan (one launch less per layer)
    scan_prep_kernel<TQ, DELTA><<<T, 256, 0, st>>>((const TQ*)q, sq, (const TQ*)k, sk, a, sa, a_bias, A_log, beta, sbeta,
                                                   beta_dt, tau_inv, aux, H, G, D);
  // the longest segment sets the step's duration: count the segments that can be about that long (a
  // prompt chunk beside many single decode rows is still one long chain)
  const long seff = max_len > 0 ? (S < (T + max_len - 1) / max_len ? S : (T + max_len - 1) / max_len) : S;
  const int lpc = D <= 128 ? 4 : (D <= 256 ? 8 : 16);
  const long blocks = seff * H * ((P + 256 / lpc - 1) / (256 / lpc));
  return dispatch_matrix_scan<TQ, DELTA>(D, blocks < 512, q, sq, k, sk, v, sv, (const float*)a, sa, (const float*)aux, state,
                                         cu, slot, pos, out, S, H, G, D, P, a_bias, A_log, beta, sbeta, beta_dt, tau_inv,
                                         one, st);
}

}  // namespace

// q, k [rows, G*D] and v [rows, H*P] slices of storage type dt (row strides sq, sk, sv); a f32 [T, H*D]
// slice (row stride sa), OVERWRITTEN with the decays; a_bias f32 [H*D]; delta != 0: A_log f32 [H], beta
// [T, >= H] slice of type beta_dt, aux f32 [T, 2*G + H] scratch; state f32 [slots, H, D, P]; out f32
// [T, H*P].  T: rows of the step (every row belongs to a segment or is padding); max_len: the longest
// segment (1: the decode form).
MX_API int mx_matrix_scan(const void* q, long sq, const void* k, long sk, const void* v, long sv, int dt, float* a,
                          long sa, const float* a_bias, const float* A_log, const void* beta, long sbeta, int beta_dt,
                          float tau, int delta, float* aux, float* state, const int* cu, const int* slot, const int* pos,
                          float* out, int S, int T, int max_len, int H, int G, int D, int P, hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  if (D < 1 || D > 512 || G < 1 || H % G || tau <= 0.f || (delta && (A_log == nullptr || beta == nullptr || aux == nullptr)))
    return (int)hipErrorInvalidValue;
  const float ti = 1.0f / tau;
  if (delta) {
    if (dt == 1)
      return run_matrix_scan<float, true>(q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt, ti, aux, state,
                                          cu, slot, pos, out, S, T, H, G, D, P, max_len, st);
    return run_matrix_scan<bf16, true>(q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt, ti, aux, state, cu,
                                       slot, pos, out, S, T, H, G, D, P, max_len, st);
  }
  if (dt == 1)
    return run_matrix_scan<float, false>(q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt, ti, aux, state,
                                         cu, slot, pos, out, S, T, H, G, D, P, max_len, st);
  return run_matrix_scan<bf16, false>(q, sq, k, sk, v, sv, a, sa, a_bias, A_log, beta, sbeta, beta_dt, ti, aux, state, cu,
                                      slot, pos, out, S, T, H, G, D, P, max_len, st);
}

// One fixed decay per head: S <- decay[h] S + act(k) act(v)^T, o = S^T act(q) * out_scale.  q, k [rows, H*D]
// slices of storage type dt_qk, v [rows, H*P] slice of type dt_v (the two may differ: rotated f32 q, k beside
// the projection's own v); act 0: none, 1: SiLU on q, k and v; decay f32 [H]; state f32 [slots, H, D, P];
// out f32 [T, H*P].  One launch, also for prompt chunks.
MX_API int mx_decay_scan(const void* q, long sq, const void* k, long sk, int dt_qk, const void* v, long sv, int dt_v,
                         int act, const float* decay, float out_scale, float* state, const int* cu, const int* slot,
                         const int* pos, float* out, int S, int T, int max_len, int H, int D, int P, hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  if (D < 1 || D > 512 || decay == nullptr || (act != 0 && act != 1)) return (int)hipErrorInvalidValue;
  const bool one = max_len == 1;
  const long seff = max_len > 0 ? (S < (T + max_len - 1) / max_len ? S : (T + max_len - 1) / max_len) : S;
  const int lpc = D <= 128 ? 4 : (D <= 256 ? 8 : 16);
  const long blocks = seff * H * ((P + 256 / lpc - 1) / (256 / lpc));
  const int code = act | (dt_v << 4);
  // v travels as an untyped pointer: the fixed mode reads it by its storage code
  if (dt_qk == 1)
    return dispatch_matrix_scan<float, 2>(D, blocks < 512, q, sq, k, sk, v, sv, (const float*)nullptr, 0L,
                                          (const float*)nullptr, state, cu, slot, pos, out, S, H, H, D, P, decay,
                                          (const float*)nullptr, (const void*)nullptr, 0L, code, out_scale, one, st);
  return dispatch_matrix_scan<bf16, 2>(D, blocks < 512, q, sq, k, sk, v, sv, (const float*)nullptr, 0L,
                                       (const float*)nullptr, state, cu, slot, pos, out, S, H, H, D, P, decay,
                                       (const float*)nullptr, (const void*)nullptr, 0L, code, out_scale, one, st);
}

// u f32 [T, R], OVERWRITTEN with the GeLU branch; z f32 [blocks, T, 2 * R / blocks], OVERWRITTEN with the gates; y [T, >= R] slice (row stride
// sy, type dt_y); state f32 [slots, R]; out [T, R] of type dt_out
MX_API int mx_lru_scan(float* u, float* z, int blocks, const float* r_bias, const float* i_bias,
                       const float* lam, const void* y, long sy, int dt_y, const float* y_bias, float* state,
                       const int* cu, const int* slot, const int* pos, void* out, int dt_out, int S, int R, int T,
                       int max_len, hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  if (blocks < 1 || R % blocks) return (int)hipErrorInvalidValue;
  if (max_len == 1) {
    const long tot = (long)S * R;
    const int g1 = (int)((tot + 255) / 256 < 8192 ? (tot + 255) / 256 : 8192);
    MX_DISPATCH(dt_y, TY, MX_DISPATCH(dt_out, TO, lru_step_kernel<TY, TO><<<g1, 256, 0, st>>>(
        u, z, R / blocks, (long)T, r_bias, i_bias, lam, (const TY*)y, sy, y_bias, state, cu, slot, pos, (TO*)out, S, R)));
    MX_RETURN_LAUNCH();
  }
  const long total = (long)T * R;
  const int gb = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
  MX_DISPATCH(dt_y, TY, lru_gates_kernel<TY><<<gb, 256, 0, st>>>(u, z, R / blocks, (long)T, r_bias, i_bias, lam, (const TY*)y,
                                                                 sy, y_bias, R));
  dim3 grid((R + LRU_CH - 1) / LRU_CH, S);
  MX_DISPATCH(dt_out, TO, lru_scan_kernel<TO><<<grid, 256, 0, st>>>(z, u, R / blocks, (long)T, state, cu, slot, pos, (TO*)out, R));
  MX_RETURN_LAUNCH();
}

// zp, xp, gp [T, >= R] slices of type dt_in (row strides sz, sx, sg): pre-activations of the update gate, of
// the candidate and of the output gate; z_bias, x_bias f32 [R] or null; ab f32 [T, 2R] and gy f32 [T, R]:
// scratch (unused by single-row steps); state f32 [slots, R]; out [T, R] of type dt_out
MX_API int mx_mingru_scan(const void* zp, long sz, const void* xp, long sx, const void* gp, long sg, int dt_in,
                          const float* z_bias, const float* x_bias, float* ab, float* gy, float* state, const int* cu,
                          const int* slot, const int* pos, void* out, int dt_out, int S, int R, int T, int max_len,
                          hipStream_t st) {
  if (S <= 0 || T <= 0) return 0;
  if (R < 1) return (int)hipErrorInvalidValue;
  if (max_len == 1) {
    const long tot = (long)S * R;
    const int g1 = (int)((tot + 255) / 256 < 8192 ? (tot + 255) / 256 : 8192);
    MX_DISPATCH(dt_in, TI, MX_DISPATCH(dt_out, TO, mingru_step_kernel<TI, TO><<<g1, 256, 0, st>>>(
        (const TI*)zp, sz, (const TI*)xp, sx, (const TI*)gp, sg, z_bias, x_bias, state, cu, slot, pos, (TO*)out, S, R)));
    MX_RETURN_LAUNCH();
  }
  if (ab == nullptr || gy == nullptr) return (int)hipErrorInvalidValue;
  const long total = (long)T * R;
  const int gb = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
  MX_DISPATCH(dt_in, TI, mingru_gates_kernel<TI><<<gb, 256, 0, st>>>((const TI*)zp, sz, (const TI*)xp, sx, (const TI*)gp, sg,
                                                                     z_bias, x_bias, ab, gy, (long)T, R));
  dim3 grid((R + LRU_CH - 1) / LRU_CH, S);
  MX_DISPATCH(dt_out, TO, lru_scan_kernel<TO><<<grid, 256, 0, st>>>(ab, gy, R, (long)T, state, cu, slot, pos, (TO*)out, R));
  MX_RETURN_LAUNCH();
}
