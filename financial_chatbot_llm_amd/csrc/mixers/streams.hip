// Several residual streams per token (hyper-connections), positional rotation of projected heads, and
// the logit scale / soft cap:
//   * mx_embed_scaled    embedding gather times a scale into `copies` equal f32 streams [T, copies, W];
//   * mx_hyper_mix       one pass over a token's streams x_1 .. x_S (f32, in place) between two sublayers:
//                            x_t <- sum_s mix[s, t] x_s + out[t] * y        (y: the sublayer output that just ran)
//                            u = sum_t in[t] x_t;   h = u / sqrt(mean(u^2) + eps) * w
//                        i.e. the write-back of one sublayer fused with the read and RMS norm of the next
//                        (S = 1, mix = out = in = 1 is the plain pre-norm residual sum);
//   * mx_rope_heads      per head of q and k: rotation of the first `rot` entries (pairs (2i, 2i+1) or
//                        (i, i + rot/2)), cos and sin times a constant, optional RMS norm over the head without
//                        a weight, a scale; q to a dense output, k to a dense output or to paged cache rows
//                        (followed by a copy of raw values into the same row);
//   * mx_logit_cap       x <- cap * tanh(x * scale / cap) (cap <= 0: the scale only), in place.
#include "mx_common.h"

namespace {

constexpr int HC_LIMIT = 16;       // streams

template <typename T>
__global__ void embed_scaled_kernel(const int* __restrict__ ids, const T* __restrict__ table, float scale, int copies,
                                    float* __restrict__ out, int W, int V) {
  const long t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  const T* row = table + (long)id * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = ldf(row + i) * scale;
    for (int c = 0; c < copies; ++c) out[(t * copies + c) * W + i] = v;
  }
}

// one block per token; the row u lives in LDS (W floats); HC_MAX: streams padded to a compile-time count
template <typename TA, typename TO, int HC_MAX>
__global__ void hyper_mix_kernel(float* __restrict__ x, const TA* __restrict__ y, long sy, const float* __restrict__ mix,
                                 const float* __restrict__ wout, const float* __restrict__ win,
                                 const float* __restrict__ w, float eps, TO* __restrict__ out, int S, int W) {
  extern __shared__ float u[];
  __shared__ float scratch[16];
  __shared__ float cm[HC_MAX * HC_MAX], co[HC_MAX], ci[HC_MAX];
  if (threadIdx.x < HC_MAX * HC_MAX) {
    const int s = threadIdx.x / HC_MAX, t = threadIdx.x % HC_MAX;
    cm[threadIdx.x] = (y != nullptr && s < S && t < S) ? mix[s * S + t] : 0.f;
    if (s == 0) {
      co[t] = (y != nullptr && t < S) ? wout[t] : 0.f;
      ci[t] = t < S ? win[t] : 0.f;
    }
  }
  __syncthreads();
  const long row = blockIdx.x;
  float* xr = x + row * S * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float xo[HC_MAX];
#pragma unroll
    for (int s = 0; s < HC_MAX; ++s) xo[s] = s < S ? xr[(long)s * W + i] : 0.f;
    float acc = 0.f;
    if (y != nullptr) {
      const float yv = ldf(y + row * sy + i);
#pragma unroll
      for (int t = 0; t < HC_MAX; ++t) {
        if (t < S) {
          float v = 0.f;
#pragma unroll
          for (int s = 0; s < HC_MAX; ++s) v += cm[s * HC_MAX + t] * xo[s];
          v += co[t] * yv;
          xr[(long)t * W + i] = v;
          acc += ci[t] * v;
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < HC_MAX; ++t) acc += ci[t] * xo[t];
    }
    u[i] = acc;
    ss += acc * acc;
  }
  if (out == nullptr) return;
  ss = mx_block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  // each thread re-reads only the entries it wrote
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + row * W + i, u[i] * r * w[i]);
}

constexpr int RH_WAVES = 4;

// one block per token, one wave per head at a time; heads 0 .. Hq-1 are q's, then k's
template <typename TI, typename TQ, typename TK>
__global__ void __launch_bounds__(RH_WAVES * 64)
rope_heads_kernel(const TI* __restrict__ q, long sq, int Hq, const TI* __restrict__ k, long sk, int Hk, int D, int rot,
                  int half, const float* __restrict__ freq, float mscale, const int* __restrict__ pos, int norm,
                  float eps, float qscale, float kscale, TQ* __restrict__ qout, TK* __restrict__ kout, long sko,
                  const int* __restrict__ slots, const TI* __restrict__ v, long sv, int nv,
                  const TI* __restrict__ vmix, long svm, float lam) {
  extern __shared__ float buf[];             // [RH_WAVES][D]
  const long t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* mine = buf + wave * D;
  const float p = (float)pos[t];
  const long krow = slots != nullptr ? slots[t] : t;
  const int hr = rot >> 1;
  for (int head = wave; head < Hq + Hk; head += RH_WAVES) {
    const bool isq = head < Hq;
    const TI* src = isq ? q + t * sq + (long)head * D : k + t * sk + (long)(head - Hq) * D;
    if (!isq && krow < 0) continue;          // wave-uniform
    float ss = 0.f;
    for (int i = lane; i < hr; i += 64) {    // a lane owns whole pairs: one sine and cosine per pair
      const int a = half ? i : 2 * i, b = half ? i + hr : 2 * i + 1;
      float sn, cs;
      sincosf(p * freq[i], &sn, &cs);
      sn *= mscale;
      cs *= mscale;
      const float u = ldf(src + a), w = ldf(src + b);
      const float ra = u * cs - w * sn, rb = w * cs + u * sn;
      mine[a] = ra;
      mine[b] = rb;
      ss += ra * ra + rb * rb;
    }
    for (int d = rot + lane; d < D; d += 64) {
      const float val = ldf(src + d);
      mine[d] = val;
      ss += val * val;
    }
    // the copy-out below reads entries other lanes wrote
    __builtin_amdgcn_wave_barrier();
    float f = isq ? qscale : kscale;
    if (norm) f *= 1.0f / sqrtf(mx_wave_sum(ss) / (float)D + eps);
    if (isq) {
      TQ* dst = qout + (t * Hq + head) * (long)D;
      for (int d = lane; d < D; d += 64) stf(dst + d, mine[d] * f);
    } else {
      TK* dst = kout + krow * sko + (long)(head - Hq) * D;
      for (int d = lane; d < D; d += 64) stf(dst + d, mine[d] * f);
    }
  }
  if (v != nullptr && krow >= 0) {
    TK* dst = kout + krow * sko + (long)Hk * D;
    if (vmix != nullptr)       // blended in f32, rounded once into the cache row
      for (int i = threadIdx.x; i < nv; i += blockDim.x)
        stf(dst + i, (1.0f - lam) * ldf(v + t * sv + i) + lam * ldf(vmix + t * svm + i));
    else
      for (int i = threadIdx.x; i < nv; i += blockDim.x) stf(dst + i, ldf(v + t * sv + i));
  }
}

template <typename T>
__global__ void logit_cap_kernel(T* __restrict__ x, float scale, float cap, long total) {
  const float inv = cap > 0.f ? 1.0f / cap : 0.f;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    float v = ldf(x + i) * scale;
    if (cap > 0.f) v = cap * tanhf(v * inv);
    stf(x + i, v);
  }
}

}  // namespace

MX_API int mx_embed_scaled(const int* ids, const void* table, int dt, float scale, int copies, float* out, int T, int W,
                           int V, hipStream_t st) {
  if (T <= 0) return 0;
  if (copies < 1) return (int)hipErrorInvalidValue;
  MX_DISPATCH(dt, TT, embed_scaled_kernel<TT><<<T, 256, 0, st>>>(ids, (const TT*)table, scale, copies, out, W, V));
  MX_RETURN_LAUNCH();
}

// x f32 [T, S, W] (updated in place when y is given); y [T, W] slice (row stride sy, type dt_y) or null;
// mix f32 [S, S] indexed [from, to], wout f32 [S] (both unused without y), win f32 [S]; w f32 [W];
// out [T, W] of type dt_out, or null (update only)
MX_API int mx_hyper_mix(float* x, const void* y, long sy, int dt_y, const float* mix, const float* wout,
                        const float* win, const float* w, float eps, void* out, int dt_out, int T, int S, int W,
                        hipStream_t st) {
  if (T <= 0) return 0;
  if (S < 1 || S > HC_LIMIT || (size_t)W * sizeof(float) > 60 * 1024 || win == nullptr ||
      (y != nullptr && (mix == nullptr || wout == nullptr)))
    return (int)hipErrorInvalidValue;
  const int nt = W >= 1024 ? 512 : 256;
  const size_t lds = (size_t)W * sizeof(float);
#define HYPER_LAUNCH(HC)                                                                                        \
  MX_DISPATCH(dt_y, TA, MX_DISPATCH(dt_out, TO, hyper_mix_kernel<TA, TO, HC><<<T, nt, lds, st>>>(                \
      x, (const TA*)y, sy, mix, wout, win, w, eps, (TO*)out, S, W)))
  if (S <= 2) HYPER_LAUNCH(2);
  else if (S <= 4) HYPER_LAUNCH(4);
  else if (S <= 8) HYPER_LAUNCH(8);
  else HYPER_LAUNCH(16);
#undef HYPER_LAUNCH
  MX_RETURN_LAUNCH();
}

// q [T, Hq*D], k [T, Hk*D] slices of type dt_in (row strides sq, sk); freq f32 [rot / 2] (rot = 0: no
// rotation); half != 0: pairs (i, i + rot/2), else (2i, 2i+1); qout [T, Hq*D] contiguous of type dt_q; kout
// rows of stride sko and type dt_k, row slots[t] (slots null: row t; a negative slot: no write); v (may be
// null): nv raw values of type dt_in copied behind the keys of the same row -- with vmix (same shape and
// type, row stride svm) as (1 - lam) v + lam vmix
MX_API int mx_rope_heads(const void* q, long sq, int Hq, const void* k, long sk, int Hk, int dt_in, int D, int rot,
                         int half, const float* freq, float mscale, const int* pos, int norm, float eps, float qscale,
                         float kscale, void* qout, int dt_q, void* kout, long sko, int dt_k, const int* slots,
                         const void* v, long sv, int nv, const void* vmix, long svm, float lam, int T,
                         hipStream_t st) {
  if (T <= 0) return 0;
  if (D < 1 || rot < 0 || rot > D || (rot & 1) || (rot > 0 && freq == nullptr) || D > 4096)
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)RH_WAVES * D * sizeof(float);
  MX_DISPATCH(dt_in, TI, MX_DISPATCH(dt_q, TQ, MX_DISPATCH(dt_k, TK, rope_heads_kernel<TI, TQ, TK>
      <<<T, RH_WAVES * 64, lds, st>>>((const TI*)q, sq, Hq, (const TI*)k, sk, Hk, D, rot, half, freq, mscale, pos, norm,
                                      eps, qscale, kscale, (TQ*)qout, (TK*)kout, sko, slots, (const TI*)v, sv, nv,
                                      (const TI*)vmix, svm, lam))));
  MX_RETURN_LAUNCH();
}

MX_API int mx_logit_cap(void* x, int dt, float scale, float cap, long total, hipStream_t st) {
  if (total <= 0) return 0;
  const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
  MX_DISPATCH(dt, TT, logit_cap_kernel<TT><<<blocks, 256, 0, st>>>((TT*)x, scale, cap, total));
  MX_RETURN_LAUNCH();
}
