// Per-row passes of the sequential (post-norm) layered decoders:
//   * embedding gather plus a hashed token-pair row, with the previous token kept per state slot;
//   * layer norm on a sublayer's OUTPUT fused with the residual add and the rounding of the next
//     GEMM input:  x <- x + LN(m) * w,  m = a  or  m = (RMSnorm(a) * wa + RMSnorm(b) * wb) / 2
//     (two mixers side by side);  without a: out = LN(x) * w (the model's last norm);
//   * gated activations act(s * gate) * (s * up) with an optional scale per row (or act alone);
//   * top-k routing on independent sigmoid (or softmax) scores;
//   * per-head RMS norm with a weight shared by the heads, times an activated gate.
#include "mx_common.h"

namespace {

constexpr int EMB_RT = 8;   // rows per block of the pair embedding

// grid (ceil(max_len / EMB_RT), S).  The block of a segment's first rows reads the slot's previous
// token and is the one that replaces it with the segment's last id (its read comes first).
template <typename T>
__global__ void embed_pairs_kernel(const int* __restrict__ ids, const T* __restrict__ table, const T* __restrict__ pairs,
                                   long mul_prev, long mul_cur, int buckets, int* __restrict__ last_token,
                                   const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ pos,
                                   float* __restrict__ out, int W, int V) {
  const int s = blockIdx.y;
  const int sl = slot[s];
  const int r0 = cu[s], n = cu[s + 1] - r0;
  const int t0 = blockIdx.x * EMB_RT;
  if (t0 >= n) return;
  int carried = 0;
  if (t0 == 0 && sl >= 0) carried = last_token[sl];
  const int t1 = min(t0 + EMB_RT, n);
  for (int i = t0; i < t1; ++i) {
    const long r = r0 + i;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= V ? V - 1 : id);
    long prow = buckets;
    if (pos[r] != 0) {
      const long prev = i > 0 ? ids[r - 1] : carried;
      prow = (prev * mul_prev + (long)ids[r] * mul_cur) % buckets;
      if (prow < 0) prow += buckets;
    }
    const T* e = table + (long)id * W;
    const T* b = pairs + prow * W;
    for (int c = threadIdx.x; c < W; c += blockDim.x) out[r * W + c] = ldf(e + c) + ldf(b + c);
  }
  if (t0 == 0 && sl >= 0) {
    __syncthreads();            // every thread of this block has read the carried token
    if (threadIdx.x == 0) last_token[sl] = ids[r0 + n - 1];
  }
}

// one block per row; the row's m lives in LDS (W floats)
template <typename TA, typename TO>
__global__ void post_norm_kernel(float* __restrict__ x, const TA* __restrict__ a, long sa, const float* __restrict__ wa,
                                 const TA* __restrict__ b, long sb, const float* __restrict__ wb,
                                 const float* __restrict__ w, float eps, TO* __restrict__ out, int W) {
  extern __shared__ float m[];
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  const float inv_w = 1.0f / (float)W;
  if (a == nullptr) {
    for (int i = threadIdx.x; i < W; i += blockDim.x) m[i] = xr[i];
  } else if (b == nullptr) {
    for (int i = threadIdx.x; i < W; i += blockDim.x) m[i] = ldf(a + t * sa + i);
  } else {
    float sa2 = 0.f, sb2 = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float u = ldf(a + t * sa + i), v = ldf(b + t * sb + i);
      sa2 += u * u;
      sb2 += v * v;
    }
    sa2 = mx_block_sum(sa2, scratch);
    sb2 = mx_block_sum(sb2, scratch);
    const float ka = 1.0f / sqrtf(sa2 * inv_w + eps), kb = 1.0f / sqrtf(sb2 * inv_w + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x)
      m[i] = 0.5f * (ldf(a + t * sa + i) * ka * wa[i] + ldf(b + t * sb + i) * kb * wb[i]);
  }
  // each thread re-reads only the entries it wrote: no barrier needed around m
  float s1 = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) s1 += m[i];
  const float mean = mx_block_sum(s1, scratch) * inv_w;
  float s2 = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float d = m[i] - mean;
    s2 += d * d;
  }
  const float k = 1.0f / sqrtf(mx_block_sum(s2, scratch) * inv_w + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float y = (m[i] - mean) * k * w[i];
    if (a == nullptr) {
      stf(out + t * W + i, y);
    } else {
      const float v = xr[i] + y;
      xr[i] = v;
      if (out != nullptr) stf(out + t * W + i, v);
    }
  }
}

// 0.5 z (1 + tanh(u)) with u = sqrt(2/pi) (z + 0.044715 z^3), written as z sigmoid(2u): one exponential
__device__ __forceinline__ float mx_gelu_tanh(float z) {
  return z * mx_sigmoid(1.5957691216057308f * (z + 0.044715f * z * z * z));
}

__device__ __forceinline__ float mx_act(float v, int act) {
  switch (act) {
    case 1: return mx_silu(v);
    case 2: return mx_gelu_tanh(v);
    case 3: return mx_sigmoid(v);
    default: return v;
  }
}

template <typename T>
__global__ void glu_act_kernel(const T* __restrict__ gate, long sg, const T* __restrict__ up, long su,
                               const float* __restrict__ row_scale, int act, T* __restrict__ out, long so, int n,
                               long total) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long t = i / n;
    const int c = (int)(i - t * n);
    const float s = row_scale != nullptr ? row_scale[t] : 1.0f;
    const float g = mx_act(s * ldf(gate + t * sg + c), act);
    stf(out + t * so + c, up != nullptr ? g * (s * ldf(up + t * su + c)) : g);
  }
}

// the same with 16-byte accesses: grid (rows, column chunks), V elements per thread; every row start and the
// column count are multiples of V elements
template <typename T, int V>
__global__ void glu_act_vec_kernel(const T* __restrict__ gate, long sg, const T* __restrict__ up, long su,
                                   const float* __restrict__ row_scale, int act, T* __restrict__ out, long so, int nv) {
  typedef T vec __attribute__((ext_vector_type(V)));
  const long t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= nv) return;
  const float s = row_scale != nullptr ? row_scale[t] : 1.0f;
  const vec g = *reinterpret_cast<const vec*>(gate + t * sg + (long)c * V);
  vec u, o;
  if (up != nullptr) u = *reinterpret_cast<const vec*>(up + t * su + (long)c * V);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float a = mx_act(s * (float)g[e], act);
    o[e] = (T)(up != nullptr ? a * (s * (float)u[e]) : a);
  }
  *reinterpret_cast<vec*>(out + t * so + (long)c * V) = o;
}

// one wave per token: the `top` largest scores (ties: the lower index) with the score as weight.
// sigmoid scores (1) keep the order of the logits; softmax scores are normalised over all E entries (0)
// or over the chosen entries only (2).
__global__ void route_scores_kernel(const float* __restrict__ z, int E, int top, int sigmoid_scores,
                                    float* __restrict__ outw, int* __restrict__ outi, int T) {
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* zr = z + (long)t * E;
  float m = -INFINITY, inv = 1.f;
  if (sigmoid_scores == 0) {
    for (int e = lane; e < E; e += 64) m = fmaxf(m, zr[e]);
    m = mx_wave_max(m);
    float s = 0.f;
    for (int e = lane; e < E; e += 64) s += expf(zr[e] - m);
    inv = 1.0f / mx_wave_sum(s);
  }
  unsigned long long taken_lo = 0, taken_hi = 0;     // this lane's entries already chosen (E <= 64 * 128)
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane, j = 0; e < E; e += 64, ++j) {
      const bool used = j < 64 ? (taken_lo >> j) & 1 : (taken_hi >> (j - 64)) & 1;
      if (used) continue;
      const float c = zr[e];
      if (c > bv || (c == bv && e < bi) || bi == 0x7fffffff) {
        bv = c;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi != 0x7fffffff && (bi & 63) == lane) {
      const int j = bi >> 6;
      if (j < 64) taken_lo |= 1ull << j; else taken_hi |= 1ull << (j - 64);
    }
    if (lane == 0) {
      const int e = bi == 0x7fffffff ? 0 : bi;
      outi[(long)t * top + k] = e;
      outw[(long)t * top + k] = bi == 0x7fffffff ? 0.f : (sigmoid_scores == 1 ? mx_sigmoid(zr[e])
                                : sigmoid_scores == 2 ? zr[e] : expf(zr[e] - m) * inv);
    }
  }
  if (sigmoid_scores == 2 && lane == 0) {       // softmax over the chosen logits (the first is the largest)
    float* w = outw + (long)t * top;
    const float m2 = w[0];
    float s = 0.f;
    for (int k = 0; k < top; ++k) {
      w[k] = expf(w[k] - m2);
      s += w[k];
    }
    const float r = 1.0f / s;
    for (int k = 0; k < top; ++k) w[k] *= r;
  }
}

// grid (rows, H): head h's P outputs / rms * w[P] * act(gate); w null: no weight
template <typename TI, typename TG, typename TO>
__global__ void head_norm_gate_kernel(const TI* __restrict__ in, long si, const float* __restrict__ w, float eps,
                                      const TG* __restrict__ gate, long sg, int act, TO* __restrict__ out, int P) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const int h = blockIdx.y, H = gridDim.y;
  const TI* r = in + t * si + (long)h * P;
  float ss = 0.f;
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const float v = ldf(r + i);
    ss += v * v;
  }
  ss = mx_block_sum(ss, scratch);
  const float k = 1.0f / sqrtf(ss / (float)P + eps);
  for (int i = threadIdx.x; i < P; i += blockDim.x)
    stf(out + (t * H + h) * P + i,
        ldf(r + i) * k * (w != nullptr ? w[i] : 1.f) * mx_act(ldf(gate + t * sg + (long)h * P + i), act));
}

}  // namespace

MX_API int mx_embed_pairs(const int* ids, const void* table, const void* pairs, int dt, int mul_prev, int mul_cur,
                          int buckets, int* last_token, const int* cu, const int* slot, const int* pos, float* out,
                          int S, int max_len, int W, int V, hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (buckets < 1) return (int)hipErrorInvalidValue;
  dim3 grid((max_len + EMB_RT - 1) / EMB_RT, S);
  MX_DISPATCH(dt, TT, embed_pairs_kernel<TT><<<grid, 256, 0, st>>>(ids, (const TT*)table, (const TT*)pairs, mul_prev,
                                                                   mul_cur, buckets, last_token, cu, slot, pos, out, W, V));
  MX_RETURN_LAUNCH();
}

// x f32 [T, W].  a given: x <- x + LN(m) * w in place and, with out, out = x in type dt_out;
// m = a, or with b: (RMSnorm(a) wa + RMSnorm(b) wb) / 2 (a, b of type dt_ab, row strides sa, sb).
// a null: out = LN(x) * w.
MX_API int mx_post_norm(float* x, const void* a, long sa, const float* wa, const void* b, long sb, const float* wb,
                        int dt_ab, const float* w, float eps, void* out, int dt_out, int T, int W, hipStream_t st) {
  if (T <= 0) return 0;
  if ((size_t)W * sizeof(float) > 60 * 1024 || (a == nullptr && out == nullptr)) return (int)hipErrorInvalidValue;
  const int nt = W >= 1024 ? 512 : 256;
  MX_DISPATCH(dt_ab, TA, MX_DISPATCH(dt_out, TO, post_norm_kernel<TA, TO><<<T, nt, (size_t)W * sizeof(float), st>>>(
      x, (const TA*)a, sa, wa, (const TA*)b, sb, wb, w, eps, (TO*)out, W)));
  MX_RETURN_LAUNCH();
}

// act: 1 SiLU, 2 tanh-form GeLU; up null: the activation alone
MX_API int mx_glu_act(const void* gate, long sg, const void* up, long su, const float* row_scale, int act, void* out,
                      long so, int dt, int T, int n, hipStream_t st) {
  const long total = (long)T * n;
  if (total <= 0) return 0;
  const int V = dt == 1 ? 4 : 8;                       // elements per 16 bytes
  const bool aligned = n % V == 0 && sg % V == 0 && so % V == 0 && (up == nullptr || su % V == 0) &&
                       ((size_t)gate | (size_t)out | (size_t)up) % 16 == 0 && (size_t)n / V <= 65535u * 256u;
  if (aligned) {
    const int nv = n / V;
    dim3 grid(T, (nv + 255) / 256);
    if (dt == 1)
      glu_act_vec_kernel<float, 4><<<grid, 256, 0, st>>>((const float*)gate, sg, (const float*)up, su, row_scale, act,
                                                         (float*)out, so, nv);
    else
      glu_act_vec_kernel<bf16, 8><<<grid, 256, 0, st>>>((const bf16*)gate, sg, (const bf16*)up, su, row_scale, act,
                                                        (bf16*)out, so, nv);
    MX_RETURN_LAUNCH();
  }
  const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
  MX_DISPATCH(dt, TT, glu_act_kernel<TT><<<blocks, 256, 0, st>>>((const TT*)gate, sg, (const TT*)up, su, row_scale, act,
                                                                  (TT*)out, so, n, total));
  MX_RETURN_LAUNCH();
}

MX_API int mx_route_scores(const float* z, int E, int top, int sigmoid_scores, float* outw, int* outi, int T,
                           hipStream_t st) {
  if (T <= 0) return 0;
  if (E > 64 * 128 || top > E) return (int)hipErrorInvalidValue;
  route_scores_kernel<<<(T + 3) / 4, 256, 0, st>>>(z, E, top, sigmoid_scores, outw, outi, T);
  MX_RETURN_LAUNCH();
}

// in [T, H*P] (row stride si, type dt_in), gate [T, H*P] slice (row stride sg, type dt_gate), out [T, H*P]
// contiguous of type dt_out; w f32 [P] or null; act: 1 SiLU, 3 sigmoid
MX_API int mx_head_norm_gate(const void* in, long si, int dt_in, const float* w, float eps, const void* gate, long sg,
                             int dt_gate, int act, void* out, int dt_out, int T, int H, int P, hipStream_t st) {
  if (T <= 0) return 0;
  const int nt = P >= 256 ? 256 : (P > 64 ? 128 : 64);
  dim3 grid(T, H);
  MX_DISPATCH(dt_in, TI, MX_DISPATCH(dt_gate, TG, MX_DISPATCH(dt_out, TO, head_norm_gate_kernel<TI, TG, TO>
      <<<grid, nt, 0, st>>>((const TI*)in, si, w, eps, (const TG*)gate, sg, act, (TO*)out, P))));
  MX_RETURN_LAUNCH();
}
