// The 32-bit residual stream and the small per-row passes around it:
//   * embedding gather into an f32 stream;
//   * parallel-block residual update fused with the next RMS norm:
//         x <- x + mult * (a + b);  y = x / sqrt(mean(x^2) + eps) * w
//     optionally with a weight per sublayer output and a sigmoid gate per element on the update:
//         x <- x + sigmoid(gate + gate_bias) * (mult_a * a + mult_b * b)
//   * RMS norm of a strided row slice (latent norms), optionally in equal groups and with a SiLU
//     gate applied first (the state-space mixer's output norm);
//   * activations: relu^2, and the clamped gated unit g * sigmoid(alpha g) * (u + 1);
//   * biased top-k routing: softmax scores, choice = score + bias, weights = unbiased scores;
//   * weighted combine of routed expert rows, identity experts and a shared expert.
#include "mx_common.h"

namespace {

template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out,
                             int W, int V) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  const T* row = table + (long)id * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) out[(long)t * W + i] = ldf(row + i);
}

// one block per row.  a / b: the two sublayer outputs of a parallel block (either may be null);
// gate (may be null): pre-activations of a sigmoid gate on the update, gate_bias f32 [W] or null.
template <typename TA, typename TO>
__global__ void residual_norm_kernel(float* __restrict__ x, const TA* __restrict__ a, long sa,
                                     const TA* __restrict__ b, long sb, float mult, float mult_b,
                                     const TA* __restrict__ gate, long sg, const float* __restrict__ gate_bias,
                                     const float* __restrict__ w, float eps, TO* __restrict__ out, int W) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  float* xr = x + t * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = xr[i];
    if (a != nullptr || b != nullptr) {
      float s;
      if (mult == mult_b) {
        s = 0.f;
        if (a != nullptr) s += ldf(a + t * sa + i);
        if (b != nullptr) s += ldf(b + t * sb + i);
        s *= mult;
      } else {
        s = (a != nullptr ? mult * ldf(a + t * sa + i) : 0.f) + (b != nullptr ? mult_b * ldf(b + t * sb + i) : 0.f);
      }
      if (gate != nullptr) s *= mx_sigmoid(ldf(gate + t * sg + i) + (gate_bias != nullptr ? gate_bias[i] : 0.f));
      v = v + s;
      xr[i] = v;
    }
    ss += v * v;
  }
  if (out == nullptr) return;
  ss = mx_block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + t * W + i, xr[i] * r * w[i]);
}

// grid (rows, groups): RMS norm of `n` contiguous elements per group.  gate (optional): the
// element is multiplied by silu(gate) BEFORE the statistics.
template <typename TI, typename TG, typename TO>
__global__ void group_norm_kernel(const TI* __restrict__ in, long si, const TG* __restrict__ gate, long sg,
                                  const float* __restrict__ w, float eps, TO* __restrict__ out, long so, int n) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const int g = blockIdx.y;
  const TI* r = in + t * si + (long)g * n;
  const TG* z = gate == nullptr ? nullptr : gate + t * sg + (long)g * n;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = ldf(r + i);
    if (z != nullptr) v *= mx_silu(ldf(z + i));
    ss += v * v;
  }
  ss = mx_block_sum(ss, scratch);
  const float k = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = ldf(r + i);
    if (z != nullptr) v *= mx_silu(ldf(z + i));
    stf(out + t * so + (long)g * n + i, v * k * w[(long)g * n + i]);
  }
}

template <typename T>
__global__ void relu2_kernel(const T* __restrict__ in, long si, T* __restrict__ out, long so, int n, long total) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long t = i / n;
    const int c = (int)(i - t * n);
    const float v = fmaxf(ldf(in + t * si + c), 0.f);
    stf(out + t * so + c, v * v);
  }
}

// gate and up are column slices (row strides sg / su) of one projection output
template <typename T>
__global__ void glu_clamp_kernel(const T* __restrict__ gate, long sg, const T* __restrict__ up, long su,
                                 float limit, float alpha, T* __restrict__ out, long so, int n, long total) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long t = i / n;
    const int c = (int)(i - t * n);
    const float g = fminf(ldf(gate + t * sg + c), limit);
    const float u = fminf(fmaxf(ldf(up + t * su + c), -limit), limit);
    stf(out + t * so + c, g * mx_sigmoid(alpha * g) * (u + 1.0f));
  }
}

// one wave per token: scores = softmax(z) over all E entries; the `top` largest score + bias are
// chosen (ties: the lower index), each with its unbiased score as weight.
__global__ void route_biased_kernel(const float* __restrict__ z, const float* __restrict__ bias, int E, int top,
                                    float* __restrict__ outw, int* __restrict__ outi, int T) {
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= T) return;
  const float* zr = z + (long)t * E;
  float m = -INFINITY;
  for (int e = lane; e < E; e += 64) m = fmaxf(m, zr[e]);
  m = mx_wave_max(m);
  float s = 0.f;
  for (int e = lane; e < E; e += 64) s += expf(zr[e] - m);
  s = mx_wave_sum(s);
  const float inv = 1.0f / s;
  unsigned long long taken_lo = 0, taken_hi = 0;     // this lane's entries already chosen (E <= 64 * 128)
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane, j = 0; e < E; e += 64, ++j) {
      const bool used = j < 64 ? (taken_lo >> j) & 1 : (taken_hi >> (j - 64)) & 1;
      if (used) continue;
      const float c = expf(zr[e] - m) * inv + (bias != nullptr ? bias[e] : 0.f);
      if (c > bv || (c == bv && e < bi)) {
        bv = c;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
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
      outw[(long)t * top + k] = bi == 0x7fffffff ? 0.f : expf(zr[e] - m) * inv;
    }
  }
}

// out[t] = sum_k w[t,k] * src(t,k) (+ shared[t]):  src is the token's own input row h[t] for an
// identity expert (index >= E), else row pos[t,k] of the expert-sorted outputs ys.
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ ys, const int* __restrict__ pos, const int* __restrict__ idx,
                                   const float* __restrict__ wts, const T* __restrict__ h, long sh,
                                   const T* __restrict__ shared, long ssh, int E, int top, int W,
                                   T* __restrict__ out) {
  const long t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float acc = shared != nullptr ? ldf(shared + t * ssh + c) : 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = idx[t * top + k];
      const float w = wts[t * top + k];
      if (w == 0.f) continue;
      const float v = e >= E ? ldf(h + t * sh + c) : ldf(ys + (long)pos[t * top + k] * W + c);
      acc += w * v;
    }
    stf(out + t * W + c, acc);
  }
}

}  // namespace

MX_API int mx_embed(const int* ids, const void* table, int dt, float* out, int T, int W, int V, hipStream_t st) {
  if (T <= 0) return 0;
  MX_DISPATCH(dt, TT, embed_kernel<TT><<<T, 256, 0, st>>>(ids, (const TT*)table, out, W, V));
  MX_RETURN_LAUNCH();
}

// x [T, W] f32 (updated in place when a or b is given); out (may be null: update only) of type dt_out;
// a, b and gate (a [T, >= W] slice, or null) of type dt_ab; mult weighs a, mult_b weighs b
MX_API int mx_residual_norm(float* x, const void* a, long sa, const void* b, long sb, int dt_ab, float mult,
                            float mult_b, const void* gate, long sg, const float* gate_bias, const float* w, float eps,
                            void* out, int dt_out, int T, int W, hipStream_t st) {
  if (T <= 0) return 0;
  const int nt = W >= 1024 ? 512 : 256;
  MX_DISPATCH(dt_ab, TA, MX_DISPATCH(dt_out, TO, residual_norm_kernel<TA, TO><<<T, nt, 0, st>>>(
      x, (const TA*)a, sa, (const TA*)b, sb, mult, mult_b, (const TA*)gate, sg, gate_bias, w, eps, (TO*)out, W)));
  MX_RETURN_LAUNCH();
}

// in [T, groups * n] (row stride si, type dt_in; f32 when dt_in == 1), optional gate of type dt_gate
MX_API int mx_group_norm(const void* in, long si, int dt_in, const void* gate, long sg, int dt_gate, const float* w,
                         float eps, void* out, long so, int dt_out, int T, int groups, int n, hipStream_t st) {
  if (T <= 0) return 0;
  const int nt = n >= 1024 ? 512 : (n >= 256 ? 256 : 64);
  dim3 grid(T, groups);
  MX_DISPATCH(dt_in, TI, MX_DISPATCH(dt_gate, TG, MX_DISPATCH(dt_out, TO, group_norm_kernel<TI, TG, TO>
      <<<grid, nt, 0, st>>>((const TI*)in, si, (const TG*)gate, sg, w, eps, (TO*)out, so, n))));
  MX_RETURN_LAUNCH();
}

MX_API int mx_relu2(const void* in, long si, void* out, long so, int dt, int T, int n, hipStream_t st) {
  const long total = (long)T * n;
  if (total <= 0) return 0;
  const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
  MX_DISPATCH(dt, TT, relu2_kernel<TT><<<blocks, 256, 0, st>>>((const TT*)in, si, (TT*)out, so, n, total));
  MX_RETURN_LAUNCH();
}

MX_API int mx_glu_clamp(const void* gate, long sg, const void* up, long su, float limit, float alpha, void* out,
                        long so, int dt, int T, int n, hipStream_t st) {
  const long total = (long)T * n;
  if (total <= 0) return 0;
  const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
  MX_DISPATCH(dt, TT, glu_clamp_kernel<TT><<<blocks, 256, 0, st>>>((const TT*)gate, sg, (const TT*)up, su, limit,
                                                                    alpha, (TT*)out, so, n, total));
  MX_RETURN_LAUNCH();
}

MX_API int mx_route_biased(const float* z, const float* bias, int E, int top, float* outw, int* outi, int T,
                           hipStream_t st) {
  if (T <= 0) return 0;
  if (E > 64 * 128 || top > E) return (int)hipErrorInvalidValue;
  route_biased_kernel<<<(T + 3) / 4, 256, 0, st>>>(z, bias, E, top, outw, outi, T);
  MX_RETURN_LAUNCH();
}

MX_API int mx_moe_combine(const void* ys, const int* pos, const int* idx, const float* wts, const void* h, long sh,
                          const void* shared, long ssh, int E, int top, int W, void* out, int dt, int T,
                          hipStream_t st) {
  if (T <= 0) return 0;
  MX_DISPATCH(dt, TT, moe_combine_kernel<TT><<<T, 256, 0, st>>>((const TT*)ys, pos, idx, wts, (const TT*)h, sh,
                                                                (const TT*)shared, ssh, E, top, W, (TT*)out));
  MX_RETURN_LAUNCH();
}
