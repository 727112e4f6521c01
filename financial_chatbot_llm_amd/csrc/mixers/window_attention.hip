// Sliding-window softmax attention with grouped key/value heads over a paged row cache.
//
// The cache row of a token is [k: G*D | v: G*P] (G key/value heads of key size D and value size P).
// Query head h reads key/value head h / (H / G).  The query at position p sees the keys j of its own
// sequence with 0 <= p - j < window -- or, chunked, the keys j <= p of its own block of `window`
// positions (floor(j / window) == floor(p / window), blocks counted from position 0 of the sequence);
// score = q . k * scale; softmax and accumulation in f32; the head's output is multiplied by
// sigmoid(gate[t, h]) when a gate is given.  Rotation and norms of q and k happen before (the cache holds
// finished keys).  Two further forms of the same walk:
//   * kept first tokens (attention sinks): with keep > 0 the keys j < keep stay visible to every later
//     query whatever the window (at their true positions); the tiles that hold them are walked before the
//     window's own tiles;
//   * sigmoid weights: with a per-head bias array the weight of a visible key is
//     sigmoid(score + head_bias[h]) and the weights are NOT normalised over the keys (no softmax).
//
//   mx_qk_norm_write   RMS norm over the WHOLE query projection and over the whole key projection
//                      (all heads at once, plain weights), cache write of [normed k | v].
//   mx_window_attend   the attention, over a flat batch of segments (prompt chunks and single
//                      decoded tokens alike).
#include <stdlib.h>

#include "mx_common.h"

namespace {

constexpr int PAGE = 64;            // tokens per cache page

// first key the query at position p sees: a sliding window of `window` keys, or the start of p's block
__device__ __forceinline__ int first_key(int p, int window, int chunked) {
  return chunked ? (p / window) * window : max(0, p - window + 1);
}

// The tiles a block walks: `nsink` tiles from key 0 that hold kept first tokens and lie wholly before
// the window's first tile, then the tiles first_tile .. last_tile.  Walk index -> first key of the tile.
__device__ __forceinline__ int walk_k0(int ti, int nsink, int first_tile, int KT) {
  return (ti < nsink ? ti : first_tile + ti - nsink) * KT;
}

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
  if (qout != nullptr)       // null: the caller reads the projection's own q slice (no norm, no copy)
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
                     long sgate, int window, int chunked, int keep, const float* __restrict__ hbias, float scale,
                     T* __restrict__ out, int H, int G, int D, int P, int QT, int HB, int KT, int ldk, int ldv) {
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
  const int lo = first_key(p_first, window, chunked);
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

  const int first_tile = lo / KT;
  const int nsink = min((keep + KT - 1) / KT, first_tile);
  const int ntiles = nsink + p_last / KT - first_tile + 1;
  for (int ti = 0; ti < ntiles; ++ti) {
    const int k0 = walk_k0(ti, nsink, first_tile, KT);
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
      const bool vis = lane < rows && j <= p && (j >= first_key(p, window, chunked) || j < keep);
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
      float corr = 1.f, pj;
      if (hbias != nullptr) {                              // independent sigmoid weights, no running statistics
        pj = vis ? mx_sigmoid(sc + hbias[h]) : 0.f;
      } else {
        const float mt = mx_wave_max(sc);
        const float mn = fmaxf(m[ii], mt);
        corr = expf(m[ii] - mn);                           // exp(-inf) = 0 on the first tile
        pj = vis ? expf(sc - mn) : 0.f;
        l[ii] = l[ii] * corr + mx_wave_sum(pj);
        m[ii] = mn;
      }
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
    float gs = hbias != nullptr ? 1.0f : 1.0f / l[ii];
    if (gate != nullptr) gs *= mx_sigmoid(ldf(gate + row * sgate + h));
#pragma unroll
    for (int c = 0; c < WA_CPL; ++c) {
      const int d = lane + 64 * c;
      if (d < P) stf(out + (row * H + h) * P + d, acc[ii][c] * gs);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// bf16 on the matrix cores (v_mfma_f32_16x16x32_bf16).  A block owns 64 (row, head) pairs of one
// segment and ONE key/value head -- QT consecutive rows x HB of its query heads, 16 pairs per wave --
// and walks the key tiles of the union of their windows, KT = 32 keys at a time.  Per tile and wave:
//     S^T = K . Q^T      A: key rows from LDS (16-byte reads), B: the wave's queries, in registers
//     online softmax     the statistics of query (lane % 16) live in that lane, f32
//     O^T += V^T . P^T   A: the value tile, transposed in LDS; B: P straight from the S^T registers
//                        (the MFMA's k slots 8g+i / 8g+4+i hold keys 4g+i / 16+4g+i), as two bf16
//                        terms hi + lo so that the f32 softmax weights are not cut to 8 bits
// Feature dimensions are zero-padded to multiples of 32 (keys) / 16 (values) in LDS and registers.
// Single-row segments (decode) may split each row's key range over nsplit blocks; the parts
// (unnormalised output, running maximum, sum) are combined by window_merge_kernel.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int MKT = 32;             // keys per tile
constexpr int MLDV = MKT + 8;       // row stride of the transposed value tile

template <int KSM, int NTM>         // up to 32*KSM key dims, 16*NTM value dims
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
window_attend_mfma_kernel(const bf16* __restrict__ q, long sq, const bf16* __restrict__ cache,
                          const int* __restrict__ cu, const int* __restrict__ pos, const int* __restrict__ bt, int btw,
                          const bf16* __restrict__ gate, long sgate, int window, int chunked, int keep,
                          const float* __restrict__ hbias, float scale, bf16* __restrict__ out, int H, int G, int D,
                          int P, int QT, int HB, int nsplit, float* __restrict__ ws) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int KS = (D + 31) / 32, NT = (P + 15) / 16;
  const int ldk = KS * 32 + 8;
  bf16* kt_lds = reinterpret_cast<bf16*>(smem);                 // [MKT][ldk]
  bf16* vt_lds = kt_lds + MKT * ldk;                            // [NT*16][MLDV]
  const int rep = H / G;
  const int hblocks = (rep + HB - 1) / HB;
  const int s = blockIdx.z;
  const int r0 = cu[s], n = cu[s + 1] - r0;
  // nsplit > 1 (single-row segments): blockIdx.x is the part of the key range this block walks
  const int split = nsplit > 1 ? blockIdx.x : 0;
  const int t0 = nsplit > 1 ? 0 : blockIdx.x * QT;
  if (t0 >= n) return;
  const int nq = min(QT, n - t0);
  const int kvh = blockIdx.y / hblocks;
  const int hg0 = (blockIdx.y - kvh * hblocks) * HB;
  const int nh = min(HB, rep - hg0);
  const int h0 = kvh * rep + hg0;
  const int Wr = G * (D + P);
  const int koff = kvh * D, voff = G * D + kvh * P;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;
  const int p_first = pos[r0 + t0], p_last = pos[r0 + t0 + nq - 1];
  const int lo = first_key(p_first, window, chunked);
  // this lane's query: pair index 16 * wave + c
  const int pair = 16 * wave + c;
  const bool qok = pair < nq * nh;
  const int tq = qok ? pair / nh : 0, hh = qok ? pair - (pair / nh) * nh : 0;
  const long row = r0 + t0 + tq;
  const int h = h0 + hh;
  const int pq = qok ? pos[row] : -1;
  const int pq_lo = qok ? first_key(pq, window, chunked) : 0;
  const bool wave_live = 16 * wave < nq * nh;
  const bool sigm = hbias != nullptr;
  const float hb = (sigm && qok) ? hbias[h] : 0.f;

  bf16x8 qf[KSM];
#pragma unroll
  for (int ks = 0; ks < KSM; ++ks) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = 32 * ks + 8 * g + e;
      qf[ks][e] = (qok && d < D) ? q[row * sq + (long)h * D + d] : (bf16)0.f;
    }
  }
  f32x4 o[NTM];
#pragma unroll
  for (int nt = 0; nt < NTM; ++nt) o[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // zero the padding columns / rows once (staging only writes real elements)
  if ((D & 31) != 0 || (P & 15) != 0) {
    unsigned* z = reinterpret_cast<unsigned*>(smem);
    const int words = (MKT * ldk + NT * 16 * MLDV) / 2;
    for (int e = threadIdx.x; e < words; e += 256) z[e] = 0u;
  }

  const int first_tile = lo / MKT;
  const int nsink = min((keep + MKT - 1) / MKT, first_tile);
  int t_begin = 0, t_end = nsink + p_last / MKT - first_tile;     // walk indices, inclusive
  if (nsplit > 1) {
    const int per = (t_end + nsplit) / nsplit;                    // ceil((t_end + 1) / nsplit)
    t_begin = split * per;
    t_end = min(t_end, t_begin + per - 1);
  }
  // staging, 16-byte path (D, P multiples of 8): a work item is a pair of keys x 8 dims of the key
  // part or of the value part -- two row loads; key pieces go to the key tile as two 16-byte stores,
  // value pieces to the transposed value tile as eight 4-byte stores (one key pair each).  The next
  // tile's loads are issued before the current tile's MFMAs and land in registers while they run.
  constexpr int MAXIT = (KSM * 32 + NTM * 16) / 8 * 16 / 256;      // 16 pairs * pieces / 256 threads
  const bool v16 = (D & 7) == 0 && (P & 7) == 0;
  const int dk8 = D >> 3, d8 = (D + P) >> 3;
  bf16x8 pre[MAXIT][2];
  auto load_tile = [&](int k0) {
    const int rows = min(MKT, p_last + 1 - k0);
    const bf16* src = cache + ((long)bt[(long)s * btw + k0 / PAGE] * PAGE + (k0 % PAGE)) * Wr;
#pragma unroll
    for (int it = 0; it < MAXIT; ++it) {
      const int e = min((int)threadIdx.x + 256 * it, 16 * d8 - 1);
      const int piece = e >> 4, jp = e & 15;
      const int col = piece < dk8 ? koff + piece * 8 : voff + (piece - dk8) * 8;
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int j = 2 * jp + r;
        bf16x8 v = *reinterpret_cast<const bf16x8*>(src + (long)min(j, rows - 1) * Wr + col);
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
        const int piece = e >> 4, jp = e & 15;
        if (piece < dk8) {
          *reinterpret_cast<bf16x8*>(kt_lds + (2 * jp) * ldk + piece * 8) = pre[it][0];
          *reinterpret_cast<bf16x8*>(kt_lds + (2 * jp + 1) * ldk + piece * 8) = pre[it][1];
        } else {
          const int d = (piece - dk8) * 8;
#pragma unroll
          for (int i = 0; i < 8; ++i)
            *reinterpret_cast<bf16x2*>(vt_lds + (d + i) * MLDV + 2 * jp) = bf16x2{pre[it][0][i], pre[it][1][i]};
        }
      }
    }
  };
  if (v16 && t_begin <= t_end) load_tile(walk_k0(t_begin, nsink, first_tile, MKT));
  for (int ti = t_begin; ti <= t_end; ++ti) {
    const int k0 = walk_k0(ti, nsink, first_tile, MKT);
    __syncthreads();
    const int rows = min(MKT, p_last + 1 - k0);
    if (v16) {
      store_tile();
    } else {
      const bf16* src = cache + ((long)bt[(long)s * btw + k0 / PAGE] * PAGE + (k0 % PAGE)) * Wr;
      for (int e = threadIdx.x; e < MKT * D; e += 256) {
        const int j = e / D, d = e - j * D;
        kt_lds[j * ldk + d] = j < rows ? src[(long)j * Wr + koff + d] : (bf16)0.f;
      }
      for (int e = threadIdx.x; e < MKT * P; e += 256) {
        const int j = e / P, d = e - j * P;
        vt_lds[d * MLDV + j] = j < rows ? src[(long)j * Wr + voff + d] : (bf16)0.f;
      }
    }
    __syncthreads();
    if (v16 && ti < t_end) load_tile(walk_k0(ti + 1, nsink, first_tile, MKT));
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
        const bool vis = j <= pq && (j >= pq_lo || j < keep);
        sc[kh][i] = vis ? st[kh][i] * scale : -INFINITY;
        tmax = fmaxf(tmax, sc[kh][i]);
      }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float mn = fmaxf(m, tmax);
    const float corr = sigm ? 1.f : ((m == -INFINITY) ? 0.f : expf(m - mn));
    // the f32 weight enters the value product as two bf16 terms, p = hi + lo (16 mantissa bits: far
    // below the rounding of the bf16 values it multiplies), both accumulated in f32
    bf16x8 pb, pl;
    float psum = 0.f;
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = sc[kh][i] == -INFINITY ? 0.f : (sigm ? mx_sigmoid(sc[kh][i] + hb) : expf(sc[kh][i] - mn));
        psum += p;
        const bf16 hi = (bf16)p;
        pb[4 * kh + i] = hi;
        pl[4 * kh + i] = (bf16)(p - (float)hi);
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
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pl, o[nt], 0, 0, 0);
      }
    }
  }
  if (!qok) return;
  if (nsplit > 1) {                          // unnormalised part: o | m | l, merged by window_merge_kernel
    float* w = ws + ((row * H + h) * nsplit + split) * (long)(P + 2);
#pragma unroll
    for (int nt = 0; nt < NTM; ++nt)
      if (nt < NT)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * nt + 4 * g + i;
          if (r < P) w[r] = o[nt][i];
        }
    if (g == 0) {
      w[P] = m;
      w[P + 1] = l;
    }
    return;
  }
  float gsc = sigm ? 1.0f : 1.0f / l;
  if (gate != nullptr) gsc *= mx_sigmoid((float)gate[row * sgate + h]);
  bf16* dst = out + (row * H + h) * P;
#pragma unroll
  for (int nt = 0; nt < NTM; ++nt) {
    if (nt < NT) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * nt + 4 * g + i;
        if (r < P) dst[r] = (bf16)(o[nt][i] * gsc);
      }
    }
  }
}

// grid (rows, H): combine the nsplit parts of one (row, head)
// (sigm: the parts are plain sums of independently weighted values)
__global__ void window_merge_kernel(const float* __restrict__ ws, const bf16* __restrict__ gate, long sgate,
                                    bf16* __restrict__ out, int H, int P, int nsplit, int sigm) {
  const long row = blockIdx.x;
  const int h = blockIdx.y;
  const float* w = ws + (row * H + h) * nsplit * (long)(P + 2);
  if (sigm) {
    const float gs = gate != nullptr ? mx_sigmoid((float)gate[row * sgate + h]) : 1.0f;
    for (int r = threadIdx.x; r < P; r += blockDim.x) {
      float a = 0.f;
      for (int i = 0; i < nsplit; ++i) a += w[i * (P + 2) + r];
      out[(row * H + h) * P + r] = (bf16)(a * gs);
    }
    return;
  }
  float M = -INFINITY;
  for (int i = 0; i < nsplit; ++i) M = fmaxf(M, w[i * (P + 2) + P]);
  float L = 0.f;
  for (int i = 0; i < nsplit; ++i) {
    const float mi = w[i * (P + 2) + P];
    if (mi != -INFINITY) L += w[i * (P + 2) + P + 1] * expf(mi - M);
  }
  float gsc = 1.0f / L;
  if (gate != nullptr) gsc *= mx_sigmoid((float)gate[row * sgate + h]);
  for (int r = threadIdx.x; r < P; r += blockDim.x) {
    float a = 0.f;
    for (int i = 0; i < nsplit; ++i) {
      const float mi = w[i * (P + 2) + P];
      if (mi != -INFINITY) a += w[i * (P + 2) + r] * expf(mi - M);
    }
    out[(row * H + h) * P + r] = (bf16)(a * gsc);
  }
}

}  // namespace

// MX_ATTEND_MFMA=0 keeps every call on the f32-lane kernel (A/B and debugging)
static bool wa_use_mfma() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("MX_ATTEND_MFMA");
    v = (e != nullptr && e[0] == '0') ? 0 : 1;
  }
  return v == 1;
}

// q [T, nq], k [T, nk], v [T, nv] slices (row strides sq, sk, sv); qw [nq], kw [nk] f32 (null: no norm);
// cache [pages*64, nk + nv]; qout [T, nq] contiguous, or null without a query norm (cache write only); all of
// storage type dt
MX_API int mx_qk_norm_write(const void* q, long sq, const void* k, long sk, const void* v, long sv, const float* qw,
                            const float* kw, float eps, const int* slots, void* cache, void* qout, int dt, int T,
                            int nq, int nk, int nv, hipStream_t st) {
  if (T <= 0) return 0;
  if (qout == nullptr && qw != nullptr) return (int)hipErrorInvalidValue;
  MX_DISPATCH(dt, TT, qk_norm_write_kernel<TT><<<T, 256, 0, st>>>((const TT*)q, sq, (const TT*)k, sk, (const TT*)v, sv, qw,
                                                                  kw, eps, slots, (TT*)cache, (TT*)qout, nq, nk, nv));
  MX_RETURN_LAUNCH();
}

// q [T, H*D] (row stride sq), out [T, H*P] contiguous; cu [S+1] row bounds of the segments, pos [T]
// positions, bt [S, btw] page tables; gate [T, >= H] slice (row stride sgate) or null.
// chunked != 0: `window` is the block size of the chunked mask instead of a sliding window's length.
// keep > 0: the first `keep` keys of the sequence stay visible beyond the window.  head_bias (f32 [H], or
// null): sigmoid weights sigmoid(score + head_bias[h]) without normalisation instead of a softmax.
// nsplit > 1 with a workspace ws (f32 [T, H, nsplit, P + 2]) and single-row segments: the key range of
// each row is walked by nsplit blocks and merged (bf16 matrix-core form only; ignored otherwise).
MX_API int mx_window_attend(const void* q, long sq, const void* cache, const int* cu, const int* pos, const int* bt,
                            int btw, const void* gate, long sgate, int window, int chunked, int keep,
                            const float* head_bias, float scale, void* out, int dt, int S, int max_len, int H, int G,
                            int D, int P, int nsplit, float* ws, hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (P > 64 * WA_CPL || G < 1 || H % G || window < 1 || keep < 0) return (int)hipErrorInvalidValue;
  const int rep = H / G;
  if (dt == 0 && D <= 256 && P <= 256 && wa_use_mfma()) {
    // matrix-core form: 64 (row, head) pairs of one key/value head per block
    const int HB = rep < 64 ? rep : 64;
    const int QT = max_len == 1 ? 1 : (64 / HB > 0 ? 64 / HB : 1);
    const int KS = (D + 31) / 32, NT = (P + 15) / 16;
    const size_t lds = ((size_t)MKT * (KS * 32 + 8) + (size_t)NT * 16 * MLDV) * sizeof(bf16);
    if (max_len != 1 || ws == nullptr || nsplit < 1) nsplit = 1;
    dim3 grid(nsplit > 1 ? nsplit : (max_len + QT - 1) / QT, G * ((rep + HB - 1) / HB), S);
    if (D <= 128 && P <= 128)
      window_attend_mfma_kernel<4, 8><<<grid, 256, lds, st>>>(
          (const bf16*)q, sq, (const bf16*)cache, cu, pos, bt, btw, (const bf16*)gate, sgate, window, chunked, keep,
          head_bias, scale, (bf16*)out, H, G, D, P, QT, HB, nsplit, ws);
    else
      window_attend_mfma_kernel<8, 16><<<grid, 256, lds, st>>>(
          (const bf16*)q, sq, (const bf16*)cache, cu, pos, bt, btw, (const bf16*)gate, sgate, window, chunked, keep,
          head_bias, scale, (bf16*)out, H, G, D, P, QT, HB, nsplit, ws);
    if (nsplit > 1) {
      dim3 g2(S, H);           // single-row segments: row index == segment index
      window_merge_kernel<<<g2, P >= 128 ? 128 : 64, 0, st>>>(ws, (const bf16*)gate, sgate, (bf16*)out, H, P, nsplit,
                                                              head_bias != nullptr ? 1 : 0);
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
      (const TT*)q, sq, (const TT*)cache, cu, pos, bt, btw, (const TT*)gate, sgate, window, chunked, keep, head_bias,
      scale, (TT*)out, H, G, D, P, QT, HB, KT, ldk, ldv));
  MX_RETURN_LAUNCH();
}
