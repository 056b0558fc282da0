// Causal attention of one row against paged caches, with everything between the dot product
// and the softmax as parameters, and the kernels that prepare its operands:
//
//   sm_rotate_heads     interleaved rotary, in place: the pair (x[2i], x[2i+1]) of every head's
//                       slice [off, off + dims) turns by the angle position * inv_freq[i]
//   sm_latent_write     a latent-attention layer's cached row: [ RMS-normed latent | shared key
//                       part, rotated ] from the down projection's output into the paged cache
//   sm_head_norm_write  q / k RMS norm per head with a weight shared by the heads: q in place,
//                       normed k and plain v into their paged caches
//   sm_row_norm_write   q / k RMS norm over the WHOLE projection (all heads at once) with weights
//                       of that size: q in place, normed k into the key cache and k as projected
//                       into the value cache (the values are the un-normalised keys)
//   sm_row_attn         for every row t at position p and every query head h
//        s_h(j)  = (q1_h . k_g(j)[0:D1] + q2_h . k_g(j)[D1:D1+D2]) * scale * temp(p)
//        s_h(j) <- cap * tanh(s_h(j) / cap)                       (cap > 0)
//        s_h(j) <- s_h(j) - r1_h * log(1 + r2_h * (p - j))        (r1 given)
//        s_h(j) <- s_h(j) - slope_h * (p - j)                     (slopes given)
//        s_h(j) <- sum_h' talk[h, h'] s_h'(j)                     (talk given)
//        o_h     = sum_{j seen} exp(s_h(j)) v_g(j) / (sum_{j seen} exp(s_h(j)) + exp(sink_h))
//        o_h    <- o_h * sigmoid(gate[t, h])                      (gate given)
//     With `sigb` there is no softmax: o_h = sum_{j seen} sigmoid(s_h(j) + sigb_h) v_g(j), the
//     weights as they are (no maximum is tracked; the running sum stays 1 so that the epilogue
//     and the merge of key splits divide by 1).  With `vdiv` > 1 the value head of key head g is
//     g / vdiv: several score maps (key heads) over one set of values.
//     with temp(p) = 1 + tcoef * log(floor((p + 1) / tevery) + 1), g = h / (H / G), and the
//     exp(sink_h) term only when a sink is given.  A row sees the keys j <= p; with a window > 0
//     only those with p - j < window and, besides them, the first `keep` keys of the sequence: the
//     64-key tiles that hold neither are skipped, so a row's cost is bounded by window + keep.  The query may come in two parts (two
//     pointers with their own strides) that face the two parts of a key row; the value cache may
//     be the key cache itself (a prefix of the key row is the value).  With G = 1 and D2 > 0 this
//     is attention over a shared compressed key / value row (the query projected into the latent
//     space beforehand); with G > 1 it is grouped-query attention.
//
// One workgroup of four waves per (row, block of HB heads): a row is a row, whether it belongs
// to a prompt's portion or is a decoded token, so its result cannot depend on how a step was
// cut.  When a step has few rows (decoding), a row's 64-key tiles are dealt out to `nsplit`
// workgroups whose partial (max, sum, accumulator) a small second kernel merges, so that the chip
// is filled whatever the batch.  Keys are visited 64 at a time, lane = key.  The waves share the heads of the block out
// among themselves (consecutive ones each): a wave scores its heads against the tile, the scores of
// all heads meet in LDS (double-buffered, one barrier per tile) where the head mixing reads
// them, then every wave runs the online softmax and the value pass of its own heads; lanes own
// 8 output channels of one key group in the value pass (16-byte loads).  Scores, weights, sums
// and angles are fp32; 16-bit types only appear at loads and stores.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kWaves = 4;
constexpr int kMaxDv = 512;
constexpr int kQPad = 8;      // padding of the 16-bit query rows in LDS (bank spread)

// v_mfma_f32_16x16x32: lane l holds A[m = l & 15][k = 8 (l >> 4) + 0..7] and
// B[k = 8 (l >> 4) + 0..7][n = l & 15]; the accumulator register i is C[4 (l >> 4) + i][l & 15]
typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8r __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8r __attribute__((ext_vector_type(8)));
template <typename T> struct Mma16 { static constexpr bool ok = false; };
template <> struct Mma16<bf16> {
  static constexpr bool ok = true;
  static __device__ __forceinline__ f32x4v run(uint4 a, uint4 b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8r, a),
                                                   __builtin_bit_cast(bf16x8r, b), c, 0, 0, 0);
  }
};
template <> struct Mma16<fp16> {
  static constexpr bool ok = true;
  static __device__ __forceinline__ f32x4v run(uint4 a, uint4 b, f32x4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8r, a),
                                                  __builtin_bit_cast(f16x8r, b), c, 0, 0, 0);
  }
};
template <> struct Mma16<float> {
  static constexpr bool ok = false;
  static __device__ __forceinline__ f32x4v run(uint4, uint4, f32x4v c) { return c; }
};

template <typename T>
__global__ void rotate_heads_kernel(T* __restrict__ x, long long ldr, long long ldh, int heads,
                                    int off, int dims, const float* __restrict__ inv_freq,
                                    const int* __restrict__ positions, long long n) {
  const int half = dims / 2;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int pr = (int)(i % half);
    const long long th = i / half;
    const int h = (int)(th % heads);
    const long long t = th / heads;
    const float a = (float)positions[t] * inv_freq[pr];
    float sn, cs;
    sincosf(a, &sn, &cs);
    T* p = x + t * ldr + h * ldh + off + 2 * pr;
    const float u = to_f32(p[0]), v = to_f32(p[1]);
    p[0] = from_f32<T>(u * cs - v * sn);
    p[1] = from_f32<T>(v * cs + u * sn);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
latent_write_kernel(const T* __restrict__ z, long long ldz, const float* __restrict__ wn,
                    const float* __restrict__ inv_freq, const int* __restrict__ positions,
                    const long long* __restrict__ slots, T* __restrict__ cache,
                    T* __restrict__ vt, int bs, int Tn, int R, int Dr, int dims, float eps) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (t >= Tn) return;
  const long long s = slots[t];
  if (s < 0) return;
  const T* zr = z + (long long)t * ldz;
  T* dst = cache + s * (R + Dr);
  float ss = 0.f;
  for (int c = lane; c < R; c += 64) {
    const float v = to_f32(zr[c]);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)R + eps);
  // vt (optional): the normed latent once more, transposed per cache block [block][R][bs], for
  // the matrix-core value product that contracts over the keys
  T* dt = vt ? vt + (s / bs) * (long long)R * bs + s % bs : nullptr;
  for (int c = lane; c < R; c += 64) {
    const T v = from_f32<T>(to_f32(zr[c]) * inv * wn[c]);
    dst[c] = v;
    if (dt) dt[(long long)c * bs] = v;
  }
  const float pos = (float)positions[t];
  for (int pr = lane; pr < dims / 2; pr += 64) {
    float sn, cs;
    sincosf(pos * inv_freq[pr], &sn, &cs);
    const float u = to_f32(zr[R + 2 * pr]), v = to_f32(zr[R + 2 * pr + 1]);
    dst[R + 2 * pr] = from_f32<T>(u * cs - v * sn);
    dst[R + 2 * pr + 1] = from_f32<T>(v * cs + u * sn);
  }
  for (int c = dims + lane; c < Dr; c += 64) dst[R + c] = zr[R + c];
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
head_norm_write_kernel(T* __restrict__ qkv, long long ld, const float* __restrict__ wq,
                       const float* __restrict__ wk, const long long* __restrict__ slots,
                       T* __restrict__ kcache, T* __restrict__ vcache, int H, int G, int D, int Dv,
                       float eps) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const long long s = slots[t];
  T* row = qkv + (long long)t * ld;
  constexpr int V = VEC ? 4 : 1;                 // elements per lane and step
  for (int item = w; item < H + 2 * G; item += kWaves) {
    if (item < H + G) {
      const bool is_q = item < H;
      T* src = row + (long long)item * D;           // q heads, then k heads, are consecutive
      T* dst = is_q ? src : (s >= 0 ? kcache + (s * G + (item - H)) * D : nullptr);
      const float* wt = is_q ? wq : wk;
      float ss = 0.f;
      for (int c = V * lane; c < D; c += 64 * V) {
        if (VEC) {
          float v[4];
          load4<T>(src + c, v);
          ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        } else {
          const float v = to_f32(src[c]);
          ss += v * v;
        }
      }
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)D + eps);
      if (dst) {
        for (int c = V * lane; c < D; c += 64 * V) {
          if (VEC) {
            float v[4], ww[4];
            load4<T>(src + c, v);
            load4<float>(wt + c, ww);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = v[e] * inv * ww[e];
            store4<T>(dst + c, v);
          } else {
            dst[c] = from_f32<T>(to_f32(src[c]) * inv * wt[c]);
          }
        }
      }
    } else if (s >= 0) {
      const int g = item - H - G;
      const T* src = row + (long long)(H + G) * D + (long long)g * Dv;
      T* dst = vcache + (s * G + g) * Dv;
      for (int c = V * lane; c < Dv; c += 64 * V) {
        if (VEC) {
          float v[4];
          load4<T>(src + c, v);
          store4<T>(dst + c, v);
        } else {
          dst[c] = src[c];
        }
      }
    }
  }
}

// One workgroup per row: the sums of squares of the query part (HD entries) and of the key part
// (GD entries) are reduced over the four waves in a fixed order, then q is normed in place and the
// key goes to both caches.  VEC: 8 entries (16 bytes of a 16-bit type) per thread and step.
template <typename T, bool VEC>
__global__ void __launch_bounds__(64 * kWaves)
row_norm_write_kernel(T* __restrict__ qk, long long ld, const float* __restrict__ wq,
                      const float* __restrict__ wk, const long long* __restrict__ slots,
                      T* __restrict__ kcache, T* __restrict__ vcache, int HD, int GD, float eps) {
  __shared__ float s_red[2][kWaves];
  constexpr int V = VEC ? 8 : 1, NT = 64 * kWaves;
  const int t = blockIdx.x, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const long long s = slots[t];
  T* q = qk + (long long)t * ld;
  const T* k = q + HD;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x * V; c < HD; c += NT * V) {
    if constexpr (VEC) {
      float v[8];
      load8<T>(q + c, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) sq += v[e] * v[e];
    } else {
      const float v = to_f32(q[c]);
      sq += v * v;
    }
  }
  for (int c = threadIdx.x * V; c < GD; c += NT * V) {
    if constexpr (VEC) {
      float v[8];
      load8<T>(k + c, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) sk += v[e] * v[e];
    } else {
      const float v = to_f32(k[c]);
      sk += v * v;
    }
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (lane == 0) {
    s_red[0][w] = sq;
    s_red[1][w] = sk;
  }
  __syncthreads();
  sq = (s_red[0][0] + s_red[0][1]) + (s_red[0][2] + s_red[0][3]);
  sk = (s_red[1][0] + s_red[1][1]) + (s_red[1][2] + s_red[1][3]);
  const float iq = 1.f / sqrtf(sq / (float)HD + eps), ik = 1.f / sqrtf(sk / (float)GD + eps);
  if (s >= 0) {
    T* kd = kcache + s * GD;
    T* vd = vcache + s * GD;
    for (int c = threadIdx.x * V; c < GD; c += NT * V) {
      if constexpr (VEC) {
        *reinterpret_cast<uint4*>(vd + c) = *reinterpret_cast<const uint4*>(k + c);
        float v[8], ww[8];
        load8<T>(k + c, v);
        load8<float>(wk + c, ww);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = v[e] * ik * ww[e];
        store8<T>(kd + c, v);
      } else {
        const T raw = k[c];
        vd[c] = raw;
        kd[c] = from_f32<T>(to_f32(raw) * ik * wk[c]);
      }
    }
  }
  for (int c = threadIdx.x * V; c < HD; c += NT * V) {
    if constexpr (VEC) {
      float v[8], ww[8];
      load8<T>(q + c, v);
      load8<float>(wq + c, ww);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = v[e] * iq * ww[e];
      store8<T>(q + c, v);
    } else {
      q[c] = from_f32<T>(to_f32(q[c]) * iq * wq[c]);
    }
  }
}

// Workgroups are handed to the 8 XCDs round-robin in launch order, and every XCD has an L2 of its
// own.  Rows that follow each other in a step belong to one sequence and read the same cache
// blocks, so XCD x takes the x-th CONTIGUOUS eighth of the rows instead of every eighth row:
// workgroup b -> row start(b % 8) + b / 8 (a bijection for any row count).
__device__ __forceinline__ int xcd_row(int b, int n) {
  const int q = n / 8, r = n % 8, x = b % 8;
  return x * q + min(x, r) + b / 8;
}

template <typename T>
struct RowAttnArgs {
  const T* q1; long long q1r, q1h; int D1;
  const T* q2; long long q2r, q2h; int D2;
  const T* kc; long long krow;
  const T* vc; long long vrow; int Dv;
  T* out; long long our, ouh;
  const int* tables; int maxb;
  const int* row_seg; const int* positions;
  int H, G, HB, bs;
  float scale, softcap, tcoef; int tevery;
  const float *r1, *r2, *talk, *sink;
  const float* slopes; int window, keep;     // linear distance bias; window + kept first keys
  const T* gate; long long gater;            // per-head output gate logits [T][H], row stride
  const float* sigb; int vdiv;               // sigmoid weights' per-head bias; key heads per value head
  int nsplit; float* ws_ml; float* ws_o;     // key splits: partial (max, sum) and accumulators
};

// The 64-key tiles a row at position `pos` visits: without a window all of 0 .. pos / 64; with one
// the tiles of the first `keep` keys (as far as they lie below the window) and then those of the
// window [pos - window + 1, pos].  Every visited tile holds at least one key the row sees.
struct TileWalk {
  int head, first, count;                    // tiles 0 .. head - 1, then first, first + 1, ...
  __device__ __forceinline__ TileWalk(int pos, int window, int keep) {
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    first = lo / 64;
    head = min((min(keep, lo) + 63) / 64, first);
    count = head + pos / 64 - first + 1;
  }
  __device__ __forceinline__ int key0(int v) const { return 64 * (v < head ? v : first + v - head); }
};
__device__ __forceinline__ bool key_seen(int j, int pos, int window, int keep) {
  return j <= pos && (window <= 0 || pos - j < window || j < keep);
}

// MMA (16-bit dtypes, key size and strides multiples of 8): the tile's scores come from the
// matrix cores as S^T = K Q^T -- wave w takes keys 16 w .. 16 w + 15 of the tile against ALL
// heads of the block, one chain of products per key/value head the block's heads use and per 16
// heads; a lane loads 16 bytes of ITS key's row per step (the contracted dimension is contiguous
// in both operands, so nothing is transposed), the queries wait in LDS in 16 bits exactly as
// projected, and the fp32 products land in the same LDS score buffer the vector path fills.
template <typename T, int HPW, bool MMA>
__global__ void __launch_bounds__(64 * kWaves)
row_attn_kernel(const RowAttnArgs<T> a) {
  extern __shared__ float smem[];
  const int t = xcd_row(blockIdx.x, gridDim.x), lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int h0 = blockIdx.y * a.HB;
  const int nh = min(a.HB, a.H - h0);
  const int Dk = a.D1 + a.D2;
  const int pos = a.positions[t];
  const int* tbl = a.tables + (long long)a.row_seg[t] * a.maxb;
  const int hpg = a.H / a.G;
  // LDS: queries (fp32 [HB][Dk], or 16-bit [16 NB][Dkp + pad]) | scores [2][HB][64] |
  // weights [HB][64] | reduction [4][kMaxDv] | cache rows of the tile's keys [2][64]
  const int Dkp = (Dk + 31) / 32 * 32;          // MMA: rows padded with zeros to the 32-wide step
  const int NB = (a.HB + 15) / 16;              // MMA: blocks of 16 heads
  float* s_q = smem;
  T* s_qb = reinterpret_cast<T*>(smem);
  float* s_sc = s_q + (MMA ? (16 * NB * (Dkp + kQPad) * (int)sizeof(T) + 3) / 4 : a.HB * Dk);
  float* s_p = s_sc + 2 * a.HB * 64;
  float* s_o = s_p + a.HB * 64;
  int* s_rb = reinterpret_cast<int*>(s_o + kWaves * kMaxDv);

  if (MMA) {
    // 8 elements (16 bytes) per thread; mma_ok guarantees the alignment of both query parts
    const int cpr = Dkp / 8;
    for (int c = threadIdx.x; c < 16 * NB * cpr; c += 64 * kWaves) {
      const int hl = c / cpr, d = (c % cpr) * 8;
      const int h = h0 + hl;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (hl < nh && d < Dk)
        v = d < a.D1
                ? *reinterpret_cast<const uint4*>(a.q1 + (long long)t * a.q1r + (long long)h * a.q1h + d)
                : *reinterpret_cast<const uint4*>(a.q2 + (long long)t * a.q2r + (long long)h * a.q2h +
                                                  (d - a.D1));
      *reinterpret_cast<uint4*>(s_qb + hl * (Dkp + kQPad) + d) = v;
    }
  } else {
    for (int i = threadIdx.x; i < nh * Dk; i += 64 * kWaves) {
      const int hl = i / Dk, d = i % Dk;
      const int h = h0 + hl;
      s_q[i] = d < a.D1 ? to_f32(a.q1[(long long)t * a.q1r + (long long)h * a.q1h + d])
                        : to_f32(a.q2[(long long)t * a.q2r + (long long)h * a.q2h + (d - a.D1)]);
    }
  }
  float temp = 1.f;
  if (a.tevery > 0 && a.tcoef != 0.f)
    temp = 1.f + a.tcoef * logf((float)((pos + 1) / a.tevery) + 1.f);
  const float qscale = a.scale * temp;

  // the wave's heads: HPW consecutive ones, so that heads of one key/value head share its rows
  const int hw0 = w * HPW;
  float m[HPW], l[HPW], acc[HPW][8], sreg[HPW];
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    const int hl = hw0 + i;
    const bool sk = a.sink != nullptr && hl < nh && blockIdx.z == 0;
    m[i] = sk ? a.sink[h0 + hl] : -INFINITY;     // the sink: a key of score sink_h, no value
    l[i] = sk ? 1.f : 0.f;
    if (a.sigb != nullptr) {                     // un-normalised weights: (m, l) = (0, 1) once
      m[i] = 0.f;
      l[i] = blockIdx.z == 0 ? 1.f : 0.f;
    }
    sreg[i] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[i][e] = 0.f;
  }
  const bool kvec = (Dk % 8 == 0) && (a.krow % 8 == 0);
  const bool vvec = (a.Dv % 8 == 0) && (a.vrow % 8 == 0);
  const int lpk = vvec ? a.Dv / 8 : 64, kpi = 64 / lpk;
  const int grp = lane / lpk, part = lane % lpk;
  const int g_lo = h0 / hpg, g_hi = (h0 + nh - 1) / hpg;          // key/value heads of the block
  __syncthreads();

  int buf = 0;
  const TileWalk walk(pos, a.window, a.keep);
  for (int tv = blockIdx.z; tv < walk.count; tv += a.nsplit, buf ^= 1) {
    const int j0 = walk.key0(tv);
    const int j = j0 + lane;
    const bool valid = key_seen(j, pos, a.window, a.keep);
    const int rb = j <= pos ? tbl[j / a.bs] * a.bs + j % a.bs : 0;
    if (w == 0) s_rb[buf * 64 + lane] = rb;
    const float dist = (float)(pos - j);
    if (MMA) {
      const int key = lane & 15, kg = lane >> 4;
      const int jk = j0 + 16 * w + key;
      const long long rbk = jk <= pos ? (long long)tbl[jk / a.bs] * a.bs + jk % a.bs : 0;
      if (16 * w <= pos - j0) {                          // the wave's 16 keys hold a visible one
        for (int g = g_lo; g <= g_hi; ++g) {
          const T* kp = a.kc + rbk * a.krow + (long long)g * Dk;
          for (int nb = 0; nb < NB; ++nb) {
            const int hl = 16 * nb + key;                // as B operand: the lane's head
            if (16 * nb >= nh || (h0 + 16 * nb) / hpg > g || (h0 + min(nh, 16 * nb + 16) - 1) / hpg < g)
              continue;                                  // none of these 16 heads uses g
            const T* qp = s_qb + hl * (Dkp + kQPad);
            f32x4v c = {0.f, 0.f, 0.f, 0.f};
            for (int d0 = 0; d0 < Dkp; d0 += 32) {
              const int d = d0 + 8 * kg;
              uint4 av = make_uint4(0u, 0u, 0u, 0u);
              if (d < Dk) av = *reinterpret_cast<const uint4*>(kp + d);
              const uint4 bv = *reinterpret_cast<const uint4*>(qp + d);
              c = Mma16<T>::run(av, bv, c);
            }
            if (hl < nh && (h0 + hl) / hpg == g) {       // c[i] = S^T[key 4 kg + i][head hl]
              const int h = h0 + hl;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const int kk = 16 * w + 4 * kg + i;
                float sv = c[i] * qscale;
                if (a.softcap > 0.f) sv = a.softcap * tanhf(sv / a.softcap);
                if (a.r1 != nullptr) sv -= a.r1[h] * logf(1.f + a.r2[h] * (float)(pos - j0 - kk));
                if (a.slopes != nullptr) sv -= a.slopes[h] * (float)(pos - j0 - kk);
                s_sc[(buf * a.HB + hl) * 64 + kk] = key_seen(j0 + kk, pos, a.window, a.keep) ? sv : 0.f;
              }
            }
          }
        }
      } else {
        for (int i = lane; i < 16 * nh; i += 64)         // no visible key: the scores are unused
          s_sc[(buf * a.HB + i / 16) * 64 + 16 * w + i % 16] = 0.f;
      }
    } else {
#pragma unroll
      for (int i = 0; i < HPW; ++i) {
        const int hl = hw0 + i;
        if (hl >= nh) break;
        const int h = h0 + hl;
        float dot = 0.f;
        if (valid) {
          const T* kp = a.kc + (long long)rb * a.krow + (long long)(h / hpg) * Dk;
          const float* qh = s_q + hl * Dk;
          if (kvec) {
            for (int d = 0; d < Dk; d += 8) {
              float kv[8];
              load8<T>(kp + d, kv);
#pragma unroll
              for (int e = 0; e < 8; ++e) dot += qh[d + e] * kv[e];
            }
          } else {
            for (int d = 0; d < Dk; ++d) dot += qh[d] * to_f32(kp[d]);
          }
        }
        float sv = dot * qscale;
        if (a.softcap > 0.f) sv = a.softcap * tanhf(sv / a.softcap);
        if (a.r1 != nullptr) sv -= a.r1[h] * logf(1.f + a.r2[h] * dist);
        if (a.slopes != nullptr) sv -= a.slopes[h] * dist;
        sv = valid ? sv : 0.f;
        sreg[i] = sv;
        s_sc[(buf * a.HB + hl) * 64 + lane] = sv;
      }
    }
    __syncthreads();
    const int nk = min(64, pos - j0 + 1);
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int hl = hw0 + i;
      if (hl >= nh) break;
      const int h = h0 + hl;
      float s = MMA ? s_sc[(buf * a.HB + hl) * 64 + lane] : sreg[i];
      if (a.talk != nullptr) {
        s = 0.f;
        for (int g = 0; g < nh; ++g) s += a.talk[h * a.H + h0 + g] * s_sc[(buf * a.HB + g) * 64 + lane];
      }
      if (a.sigb != nullptr) {
        s_p[hl * 64 + lane] = valid ? sigmoid_f(s + a.sigb[h]) : 0.f;
        continue;
      }
      s = valid ? s : -INFINITY;
      const float mn = fmaxf(m[i], wave_max(s));          // finite: a visited tile holds a seen key
      const float p = valid ? expf(s - mn) : 0.f;
      const float corr = expf(m[i] - mn);
      l[i] = l[i] * corr + wave_sum(p);
      m[i] = mn;
      s_p[hl * 64 + lane] = p;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[i][e] *= corr;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    if (hw0 < nh) {
      // value pass: a value row is loaded once for all heads of the wave that share its
      // key/value head, four rows in flight before their products
      const int gw_lo = (h0 + hw0) / hpg, gw_hi = (h0 + min(nh, hw0 + HPW) - 1) / hpg;
      for (int g = gw_lo; g <= gw_hi; ++g) {
        const T* vbase = a.vc + (long long)(g / a.vdiv) * a.Dv;
        if (vvec) {
          if (grp < kpi) {
            constexpr int U = 4;
            for (int jj = grp; jj < nk; jj += kpi * U) {
              Vec8<T> raw[U];
#pragma unroll
              for (int u = 0; u < U; ++u) {
                const int k = min(jj + u * kpi, nk - 1);
                raw[u] = *reinterpret_cast<const Vec8<T>*>(
                    vbase + (long long)s_rb[buf * 64 + k] * a.vrow + 8 * part);
              }
#pragma unroll
              for (int u = 0; u < U; ++u) {
                const int k = jj + u * kpi;
                if (k < nk) {
                  float vv[8];
#pragma unroll
                  for (int e = 0; e < 8; ++e) vv[e] = to_f32(raw[u].v[e]);
#pragma unroll
                  for (int i = 0; i < HPW; ++i) {
                    const int hl = hw0 + i;
                    if (hl < nh && (h0 + hl) / hpg == g) {
                      const float pj = s_p[hl * 64 + k];
#pragma unroll
                      for (int e = 0; e < 8; ++e) acc[i][e] += pj * vv[e];
                    }
                  }
                }
              }
            }
          }
        } else {
          for (int jj = 0; jj < nk; ++jj) {
            const T* vp = vbase + (long long)s_rb[buf * 64 + jj] * a.vrow;
            float vv[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const int d = lane + 64 * e;
              vv[e] = d < a.Dv ? to_f32(vp[d]) : 0.f;
            }
#pragma unroll
            for (int i = 0; i < HPW; ++i) {
              const int hl = hw0 + i;
              if (hl < nh && (h0 + hl) / hpg == g) {
                const float pj = s_p[hl * 64 + jj];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[i][e] += pj * vv[e];
              }
            }
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  float* so = s_o + w * kMaxDv;
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    const int hl = hw0 + i;
    if (hl >= nh) break;
    const int h = h0 + hl;
    if (vvec) {
      // sum the key groups: every group adds its 8 channels into the wave's LDS row in turn
      for (int d = lane; d < a.Dv; d += 64) so[d] = 0.f;
      for (int gq = 0; gq < kpi; ++gq) {
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        if (grp == gq) {
#pragma unroll
          for (int e = 0; e < 8; ++e) so[8 * part + e] += acc[i][e];
        }
      }
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int d = lane + 64 * e;
        if (d < a.Dv) so[d] = acc[i][e];
      }
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    }
    if (a.nsplit == 1) {
      float inv = 1.f / l[i];
      if (a.gate != nullptr) inv *= sigmoid_f(to_f32(a.gate[(long long)t * a.gater + h]));
      T* op = a.out + (long long)t * a.our + (long long)h * a.ouh;
      for (int d = lane; d < a.Dv; d += 64) op[d] = from_f32<T>(so[d] * inv);
    } else {
      // this split's running state, un-normalised; row_attn_combine merges the splits
      const long long slot = ((long long)t * a.H + h) * a.nsplit + blockIdx.z;
      if (lane == 0) {
        a.ws_ml[2 * slot] = m[i];
        a.ws_ml[2 * slot + 1] = l[i];
      }
      for (int d = lane; d < a.Dv; d += 64) a.ws_o[slot * a.Dv + d] = so[d];
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- latent attention on the matrix cores -------------------------------------------------------
// One key/value head whose value is the first Dv columns of the key row, 16-bit dtypes, Dv a
// multiple of 64, cache blocks of a multiple of 8 tokens, and a second copy `vt` of the values
// transposed per cache block, [block][Dv][bs].  A workgroup takes one row, up to 16 heads and 128
// keys per step; wave w
//   1. scores its own 32 keys against all heads: S^T = K Q^T (two 16-key tiles share the query
//      operand from LDS), scales / caps / biases / masks them and takes their maxima per head;
//   2. after the maxima of the four waves met in LDS: p = exp(s - max) for its keys, stored in LDS
//      per head as a 16-bit head plus a 16-bit remainder (~16 mantissa bits of the fp32 weight);
//   3. accumulates O^T = V^T P^T for ITS quarter of the value channels over all 128 keys: the A
//      operand is 16 bytes of `vt` (8 consecutive keys of one channel), the B operand 16 bytes of
//      the weights of one head; the accumulator's column is the head, so the running correction is
//      lane-local and nothing is merged across waves at the end.
// Scores, maxima, sums and the accumulator are fp32.
template <typename T, int NT>   // NT: 16-channel tiles per wave, Dv = 64 NT
__global__ void __launch_bounds__(64 * kWaves)
latent_attn_kernel(const RowAttnArgs<T> a, const T* __restrict__ vt) {
  extern __shared__ float smem[];
  constexpr int kPRow = 128 + 8;                 // weights per head in LDS: 128 keys + padding
  const int t = xcd_row(blockIdx.x, gridDim.x), lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int h0 = blockIdx.y * 16;
  const int nh = min(16, a.H - h0);
  const int Dk = a.D1 + a.D2;
  const int Dkp = (Dk + 31) / 32 * 32;
  const int pos = a.positions[t];
  const int* tbl = a.tables + (long long)a.row_seg[t] * a.maxb;
  const int hd = lane & 15, kg = lane >> 4;
  T* s_qb = reinterpret_cast<T*>(smem);                               // [16][Dkp + pad]
  T* s_ph = s_qb + 16 * (Dkp + kQPad);                                // [16][kPRow] head
  T* s_pl = s_ph + 16 * kPRow;                                        // [16][kPRow] remainder
  float* s_m = reinterpret_cast<float*>(s_pl + 16 * kPRow);           // [4][16]
  float* s_l = s_m + kWaves * 16;                                     // [4][16]

  const int cpr = Dkp / 8;
  for (int c = threadIdx.x; c < 16 * cpr; c += 64 * kWaves) {
    const int hl = c / cpr, d = (c % cpr) * 8;
    const int h = h0 + hl;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (hl < nh && d < Dk)
      v = d < a.D1
              ? *reinterpret_cast<const uint4*>(a.q1 + (long long)t * a.q1r + (long long)h * a.q1h + d)
              : *reinterpret_cast<const uint4*>(a.q2 + (long long)t * a.q2r + (long long)h * a.q2h +
                                                (d - a.D1));
    *reinterpret_cast<uint4*>(s_qb + hl * (Dkp + kQPad) + d) = v;
  }
  float temp = 1.f;
  if (a.tevery > 0 && a.tcoef != 0.f)
    temp = 1.f + a.tcoef * logf((float)((pos + 1) / a.tevery) + 1.f);
  const float qscale = a.scale * temp;
  const bool head_on = hd < nh;
  const int h = h0 + (head_on ? hd : 0);
  const bool sk = a.sink != nullptr && blockIdx.z == 0;
  float m_run = sk ? a.sink[h] : -INFINITY, l_run = sk ? 1.f : 0.f;
  f32x4v O[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) O[n] = f32x4v{0.f, 0.f, 0.f, 0.f};
  const T* qp = s_qb + hd * (Dkp + kQPad);
  __syncthreads();

  for (int j0 = 128 * blockIdx.z; j0 <= pos; j0 += 128 * a.nsplit) {
    // 1. scores of the wave's 32 keys
    const int jw = j0 + 32 * w;
    float sc[2][4];
    float mx = -INFINITY;
    if (jw <= pos) {
      f32x4v c0 = {0.f, 0.f, 0.f, 0.f}, c1 = {0.f, 0.f, 0.f, 0.f};
      const int k0 = min(jw + hd, pos), k1 = min(jw + 16 + hd, pos);        // addressable keys
      const T* kp0 = a.kc + ((long long)tbl[k0 / a.bs] * a.bs + k0 % a.bs) * a.krow;
      const T* kp1 = a.kc + ((long long)tbl[k1 / a.bs] * a.bs + k1 % a.bs) * a.krow;
      for (int d0 = 0; d0 < Dkp; d0 += 32) {
        const int d = d0 + 8 * kg;
        uint4 a0 = make_uint4(0u, 0u, 0u, 0u), a1 = a0;
        if (d < Dk) {
          a0 = *reinterpret_cast<const uint4*>(kp0 + d);
          a1 = *reinterpret_cast<const uint4*>(kp1 + d);
        }
        const uint4 bv = *reinterpret_cast<const uint4*>(qp + d);
        c0 = Mma16<T>::run(a0, bv, c0);
        c1 = Mma16<T>::run(a1, bv, c1);
      }
#pragma unroll
      for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = jw + 16 * sb + 4 * kg + i;         // c[i] = S^T[key 4 kg + i][head hd]
          float sv = (sb ? c1[i] : c0[i]) * qscale;
          if (a.softcap > 0.f) sv = a.softcap * tanhf(sv / a.softcap);
          if (a.r1 != nullptr) sv -= a.r1[h] * logf(1.f + a.r2[h] * (float)(pos - j));
          sv = j <= pos ? sv : -INFINITY;
          sc[sb][i] = sv;
          mx = fmaxf(mx, sv);
        }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    } else {
#pragma unroll
      for (int sb = 0; sb < 2; ++sb)
#pragma unroll
        for (int i = 0; i < 4; ++i) sc[sb][i] = -INFINITY;
    }
    if (kg == 0) s_m[w * 16 + hd] = mx;
    __syncthreads();
    // 2. the tile's maximum per head, the weights of the wave's keys into LDS
    float mt = fmaxf(fmaxf(s_m[hd], s_m[16 + hd]), fmaxf(s_m[32 + hd], s_m[48 + hd]));
    const float mn = fmaxf(m_run, mt);                     // finite: key j0 is visible
    const float corr = expf(m_run - mn);
    float ls = 0.f;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      float ph[4], pl[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = sc[sb][i] == -INFINITY ? 0.f : expf(sc[sb][i] - mn);
        ls += pv;
        ph[i] = to_f32(from_f32<T>(pv));
        pl[i] = pv - ph[i];
      }
      const int col = 32 * w + 16 * sb + 4 * kg;
      *reinterpret_cast<uint2*>(s_ph + hd * kPRow + col) = make_uint2(pk2<T>(ph[0], ph[1]), pk2<T>(ph[2], ph[3]));
      *reinterpret_cast<uint2*>(s_pl + hd * kPRow + col) = make_uint2(pk2<T>(pl[0], pl[1]), pk2<T>(pl[2], pl[3]));
    }
    ls += __shfl_xor(ls, 16, 64);
    ls += __shfl_xor(ls, 32, 64);
    if (kg == 0) s_l[w * 16 + hd] = ls;
#pragma unroll
    for (int n = 0; n < NT; ++n) O[n] *= corr;
    __syncthreads();
    // 3. O^T += V^T P^T for the wave's channels over the tile's keys
    l_run = l_run * corr + (s_l[hd] + s_l[16 + hd]) + (s_l[32 + hd] + s_l[48 + hd]);
    m_run = mn;
    for (int ks = 0; ks < 4; ++ks) {
      const int jb = j0 + 32 * ks + 8 * kg;                // the lane's 8 keys
      if (j0 + 32 * ks > pos) break;
      const uint4 bh = *reinterpret_cast<const uint4*>(s_ph + hd * kPRow + 32 * ks + 8 * kg);
      const uint4 bl = *reinterpret_cast<const uint4*>(s_pl + hd * kPRow + 32 * ks + 8 * kg);
      const int ka = min(jb, pos);
      const T* vp = vt + ((long long)tbl[ka / a.bs] * a.Dv) * a.bs + jb % a.bs;
      // keys past the row's position carry weight 0 but may hold anything: blank them
      const int nv = pos - jb + 1;                         // visible keys among the lane's 8
      uint4 mk = make_uint4(~0u, ~0u, ~0u, ~0u);
      if (nv < 8) {
        const unsigned e = nv <= 0 ? 0u : (unsigned)nv;
        const unsigned long long lo = e >= 4 ? ~0ull : (e == 0 ? 0ull : ((1ull << (16 * e)) - 1));
        const unsigned long long hi = e <= 4 ? 0ull : ((1ull << (16 * (e - 4))) - 1);
        mk = make_uint4((unsigned)lo, (unsigned)(lo >> 32), (unsigned)hi, (unsigned)(hi >> 32));
      }
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const int dv = (w * NT + n) * 16 + hd;             // as A operand: the lane's channel
        uint4 av = *reinterpret_cast<const uint4*>(vp + (long long)dv * a.bs);
        av.x &= mk.x; av.y &= mk.y; av.z &= mk.z; av.w &= mk.w;
        O[n] = Mma16<T>::run(av, bh, O[n]);
        O[n] = Mma16<T>::run(av, bl, O[n]);
      }
    }
  }
  // O[n][i] = O^T[channel (w NT + n) 16 + 4 kg + i][head hd]
  if (head_on) {
    if (a.nsplit == 1) {
      float inv = 1.f / l_run;
      if (a.gate != nullptr) inv *= sigmoid_f(to_f32(a.gate[(long long)t * a.gater + h]));
      T* op = a.out + (long long)t * a.our + (long long)h * a.ouh;
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const int dv = (w * NT + n) * 16 + 4 * kg;
        *reinterpret_cast<uint2*>(op + dv) =
            make_uint2(pk2<T>(O[n][0] * inv, O[n][1] * inv), pk2<T>(O[n][2] * inv, O[n][3] * inv));
      }
    } else {
      const long long slot = ((long long)t * a.H + h) * a.nsplit + blockIdx.z;
      if (w == 0 && kg == 0) {
        a.ws_ml[2 * slot] = m_run;
        a.ws_ml[2 * slot + 1] = l_run;
      }
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        const int dv = (w * NT + n) * 16 + 4 * kg;
        *reinterpret_cast<float4*>(a.ws_o + slot * a.Dv + dv) =
            make_float4(O[n][0], O[n][1], O[n][2], O[n][3]);
      }
    }
  }
}

inline size_t latent_attn_lds(int Dk, int esz) {
  return (size_t)16 * ((Dk + 31) / 32 * 32 + kQPad) * esz + 2 * (size_t)16 * (128 + 8) * esz +
         2 * kWaves * 16 * sizeof(float);
}

template <typename T>
hipError_t launch_latent_attn(const RowAttnArgs<T>& a, const T* vt, int Tn, hipStream_t st) {
  const size_t lds = latent_attn_lds(a.D1 + a.D2, sizeof(T));
  const dim3 grid(Tn, (a.H + 15) / 16, a.nsplit);
  switch (a.Dv / 64) {
    case 1: latent_attn_kernel<T, 1><<<grid, 64 * kWaves, lds, st>>>(a, vt); break;
    case 2: latent_attn_kernel<T, 2><<<grid, 64 * kWaves, lds, st>>>(a, vt); break;
    case 3: latent_attn_kernel<T, 3><<<grid, 64 * kWaves, lds, st>>>(a, vt); break;
    case 4: latent_attn_kernel<T, 4><<<grid, 64 * kWaves, lds, st>>>(a, vt); break;
    case 6: latent_attn_kernel<T, 6><<<grid, 64 * kWaves, lds, st>>>(a, vt); break;
    case 8: latent_attn_kernel<T, 8><<<grid, 64 * kWaves, lds, st>>>(a, vt); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}
template <>
hipError_t launch_latent_attn<float>(const RowAttnArgs<float>&, const float*, int, hipStream_t) {
  return hipErrorInvalidValue;
}

// out[t, h] = sum_s acc_s exp(m_s - M) / sum_s l_s exp(m_s - M), M = max_s m_s: the splits of a
// row's keys merged; a split that saw no key has (m, l) = (-inf, 0) and drops out.  With a gate
// the head's output is multiplied by sigmoid(gate[t, h]).
template <typename T>
__global__ void __launch_bounds__(256)
row_attn_combine_kernel(const float* __restrict__ ws_ml, const float* __restrict__ ws_o,
                        T* __restrict__ out, long long our, long long ouh, int H, int Dv,
                        int nsplit, const T* __restrict__ gate, long long gater) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63;
  const long long base = ((long long)t * H + h) * nsplit;
  __shared__ float s_w[64];
  if (threadIdx.x < 64) {                                // nsplit <= 64: lane s weighs split s
    const float ms = lane < nsplit ? ws_ml[2 * (base + lane)] : -INFINITY;
    const float ls = lane < nsplit ? ws_ml[2 * (base + lane) + 1] : 0.f;
    const float M = wave_max(ms);
    const float e = ms == -INFINITY ? 0.f : expf(ms - M);
    float L = wave_sum(ls * e);
    if (gate != nullptr) L *= 1.f + expf(-to_f32(gate[(long long)t * gater + h]));   // / sigmoid
    s_w[lane] = e / L;
  }
  __syncthreads();
  T* op = out + (long long)t * our + (long long)h * ouh;
  for (int d = threadIdx.x; d < Dv; d += 256) {
    float o = 0.f;
    for (int s = 0; s < nsplit; ++s) o += ws_o[(base + s) * Dv + d] * s_w[s];
    op[d] = from_f32<T>(o);
  }
}

inline size_t row_attn_lds(int HB, int Dk, bool mma = false, int esz = 2) {
  const size_t q = mma ? ((size_t)16 * ((HB + 15) / 16) * ((Dk + 31) / 32 * 32 + kQPad) * esz + 3) / 4 * 4
                       : sizeof(float) * (size_t)HB * Dk;
  return q + sizeof(float) * (3 * (size_t)HB * 64 + kWaves * kMaxDv) + sizeof(int) * 2 * 64;
}

template <typename T>
bool row_attn_mma_ok(const RowAttnArgs<T>& a) {
  const int Dk = a.D1 + a.D2;
  const auto al = [](const void* p) { return (uintptr_t)p % 16 == 0; };
  return Mma16<T>::ok && Dk % 8 == 0 && a.D1 % 8 == 0 && a.krow % 8 == 0 && al(a.kc) &&
         al(a.q1) && a.q1r % 8 == 0 && a.q1h % 8 == 0 &&
         (a.D2 == 0 || (al(a.q2) && a.q2r % 8 == 0 && a.q2h % 8 == 0)) &&
         row_attn_lds(a.HB, Dk, true, sizeof(T)) <= 65536;
}

template <typename T>
hipError_t launch_row_attn(const RowAttnArgs<T>& a, int Tn, hipStream_t st) {
  const int Dk = a.D1 + a.D2;
  const bool mma = row_attn_mma_ok(a);
  const size_t lds = row_attn_lds(a.HB, Dk, mma, sizeof(T));
  if (lds > 65536) return hipErrorInvalidValue;
  const dim3 grid(Tn, (a.H + a.HB - 1) / a.HB, a.nsplit);
  const int hpw = (a.HB + kWaves - 1) / kWaves;
#define LAUNCH(N, M) row_attn_kernel<T, N, M><<<grid, 64 * kWaves, lds, st>>>(a)
  if (mma) {
    if (hpw <= 1) LAUNCH(1, true);
    else if (hpw <= 2) LAUNCH(2, true);
    else if (hpw <= 4) LAUNCH(4, true);
    else if (hpw <= 8) LAUNCH(8, true);
    else return hipErrorInvalidValue;
  } else {
    if (hpw <= 1) LAUNCH(1, false);
    else if (hpw <= 2) LAUNCH(2, false);
    else if (hpw <= 4) LAUNCH(4, false);
    else if (hpw <= 8) LAUNCH(8, false);
    else return hipErrorInvalidValue;
  }
#undef LAUNCH
  if (a.nsplit > 1)
    row_attn_combine_kernel<T><<<dim3(Tn, a.H), 256, 0, st>>>(a.ws_ml, a.ws_o, a.out, a.our, a.ouh,
                                                              a.H, a.Dv, a.nsplit, a.gate, a.gater);
  return hipGetLastError();
}

inline int grid_for(long long n, int block = 256) {
  const long long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : g > 65535 ? 65535 : g);
}

}  // namespace

extern "C" {

hipError_t sm_rotate_heads(int dt, void* x, long long ldr, long long ldh, int heads, int off,
                           int dims, const float* inv_freq, const int* positions, int T,
                           hipStream_t st) {
  const long long n = (long long)T * heads * (dims / 2);
  if (n == 0) return hipSuccess;
  if (dims % 2) return hipErrorInvalidValue;
#define CALL(TT) rotate_heads_kernel<TT><<<grid_for(n), 256, 0, st>>>((TT*)x, ldr, ldh, heads, off, dims, inv_freq, positions, n)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_latent_write(int dt, const void* z, long long ldz, const float* wn,
                           const float* inv_freq, const int* positions, const long long* slots,
                           void* cache, void* vt, int bs, int T, int R, int Dr, int dims,
                           float eps, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (dims % 2 || dims > Dr) return hipErrorInvalidValue;
#define CALL(TT) latent_write_kernel<TT><<<(T + kWaves - 1) / kWaves, 256, 0, st>>>((const TT*)z, ldz, wn, inv_freq, positions, slots, (TT*)cache, (TT*)vt, bs, T, R, Dr, dims, eps)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_head_norm_write(int dt, void* qkv, long long ld, const float* wq, const float* wk,
                              const long long* slots, void* kcache, void* vcache, int T, int H,
                              int G, int D, int Dv, float eps, hipStream_t st) {
  if (T == 0) return hipSuccess;
  const bool vec = D % 4 == 0 && Dv % 4 == 0 && ld % 4 == 0 && (uintptr_t)qkv % 16 == 0 &&
                   (uintptr_t)kcache % 16 == 0 && (uintptr_t)vcache % 16 == 0 &&
                   (uintptr_t)wq % 16 == 0 && (uintptr_t)wk % 16 == 0;
#define CALL(TT)                                                                               \
  if (vec) head_norm_write_kernel<TT, true><<<T, 256, 0, st>>>((TT*)qkv, ld, wq, wk, slots,   \
                                                (TT*)kcache, (TT*)vcache, H, G, D, Dv, eps);   \
  else head_norm_write_kernel<TT, false><<<T, 256, 0, st>>>((TT*)qkv, ld, wq, wk, slots,      \
                                                 (TT*)kcache, (TT*)vcache, H, G, D, Dv, eps)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

// qk [T, >= HD + GD] (row stride ld): q normed in place over its HD entries with wq [HD]; the key
// part normed with wk [GD] into kcache and copied as projected into vcache, both [rows, GD].
hipError_t sm_row_norm_write(int dt, void* qk, long long ld, const float* wq, const float* wk,
                             const long long* slots, void* kcache, void* vcache, int T, int HD,
                             int GD, float eps, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (HD < 1 || GD < 1 || ld < HD + GD) return hipErrorInvalidValue;
  // 16-byte accesses: 16-bit dtypes, every part a multiple of 8 entries, aligned bases
  const bool vec = dt != kF32 && HD % 8 == 0 && GD % 8 == 0 && ld % 8 == 0 &&
                   (uintptr_t)qk % 16 == 0 && (uintptr_t)kcache % 16 == 0 &&
                   (uintptr_t)vcache % 16 == 0 && (uintptr_t)wq % 16 == 0 && (uintptr_t)wk % 16 == 0;
#define CALL(TT)                                                                                \
  if (vec) row_norm_write_kernel<TT, true><<<T, 64 * kWaves, 0, st>>>(                          \
      (TT*)qk, ld, wq, wk, slots, (TT*)kcache, (TT*)vcache, HD, GD, eps);                       \
  else row_norm_write_kernel<TT, false><<<T, 64 * kWaves, 0, st>>>(                             \
      (TT*)qk, ld, wq, wk, slots, (TT*)kcache, (TT*)vcache, HD, GD, eps)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

// 1 when sm_latent_attn has a kernel for these sizes (dtype code dt, value size Dv = the latent,
// key size Dk, cache block bs), else 0: the caller then takes sm_row_attn
int sm_latent_attn_ok(int dt, int Dv, int Dk, int D1, int bs) {
  if (dt != kBF16 && dt != kF16) return 0;
  const int nt = Dv / 64;
  return Dv % 64 == 0 && (nt == 1 || nt == 2 || nt == 3 || nt == 4 || nt == 6 || nt == 8) &&
         Dk % 8 == 0 && D1 % 8 == 0 && Dv <= Dk && bs % 8 == 0 && latent_attn_lds(Dk, 2) <= 65536;
}

// Latent attention (one key/value head, values = the first Dv columns of a key row) with the
// value product on the matrix cores; `vt` is the per-block transposed copy of the values that
// sm_latent_write keeps.  Arguments as sm_row_attn (no head mixing); strides of q and out must be
// multiples of 8 / 4 elements.
hipError_t sm_latent_attn(int dt, const void* q1, long long q1r, long long q1h, int D1,
                          const void* q2, long long q2r, long long q2h, int D2, const void* kc,
                          long long krow, const void* vt, int Dv, void* out, long long our,
                          long long ouh, const int* tables, int maxb, const int* row_seg,
                          const int* positions, int T, int H, int bs, float scale, float softcap,
                          float tcoef, int tevery, const float* r1, const float* r2,
                          const float* sink, const void* gate, long long gater, int nsplit,
                          float* ws_ml, float* ws_o, hipStream_t st) {
  if (T == 0) return hipSuccess;
  const auto al = [](const void* p) { return (uintptr_t)p % 16 == 0; };
  if (!sm_latent_attn_ok(dt, Dv, D1 + D2, D1, bs) || nsplit < 1 || nsplit > 64 ||
      (nsplit > 1 && (!ws_ml || !ws_o)) || krow % 8 || !al(kc) || !al(vt) || !al(q1) || q1r % 8 ||
      q1h % 8 || (D2 > 0 && (!q2 || !al(q2) || q2r % 8 || q2h % 8)) || our % 4 || ouh % 4 ||
      (uintptr_t)out % 8)
    return hipErrorInvalidValue;
#define CALL(TT)                                                                              \
  {                                                                                           \
    RowAttnArgs<TT> a{(const TT*)q1, q1r, q1h, D1, (const TT*)q2, q2r, q2h, D2,               \
                      (const TT*)kc, krow, (const TT*)kc, krow, Dv, (TT*)out, our, ouh,       \
                      tables, maxb, row_seg, positions, H, 1, 16, bs, scale, softcap, tcoef,  \
                      tevery, r1, r2, nullptr, sink, nullptr, 0, 0, (const TT*)gate, gater,   \
                      nullptr, 1, nsplit, ws_ml, ws_o};                                       \
    hipError_t e = launch_latent_attn<TT>(a, (const TT*)vt, T, st);                           \
    if (e != hipSuccess) return e;                                                            \
    if (nsplit > 1)                                                                           \
      row_attn_combine_kernel<TT><<<dim3(T, H), 256, 0, st>>>(                                \
          ws_ml, ws_o, (TT*)out, our, ouh, H, Dv, nsplit, (const TT*)gate, gater);            \
    return hipGetLastError();                                                                 \
  }
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

// LDS bytes a (HB heads, key size Dk) block needs; the caller picks HB so that this fits 64 KB
int sm_row_attn_lds(int HB, int Dk) { return (int)row_attn_lds(HB, Dk, false); }

hipError_t sm_row_attn(int dt, const void* q1, long long q1r, long long q1h, int D1,
                       const void* q2, long long q2r, long long q2h, int D2, const void* kc,
                       long long krow, const void* vc, long long vrow, int Dv, void* out,
                       long long our, long long ouh, const int* tables, int maxb,
                       const int* row_seg, const int* positions, int T, int H, int G, int HB,
                       int bs, float scale, float softcap, float tcoef, int tevery,
                       const float* r1, const float* r2, const float* talk, const float* sink,
                       const float* slopes, int window, int keep, const void* gate,
                       long long gater, const float* sigb, int vdiv, int nsplit, float* ws_ml,
                       float* ws_o, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && (!ws_ml || !ws_o))) return hipErrorInvalidValue;
  if (vdiv < 1 || G % vdiv != 0 || (sigb && sink)) return hipErrorInvalidValue;
  if (H % G != 0 || HB < 1 || HB > 8 * kWaves || Dv > kMaxDv || (talk && HB < H) ||
      (D2 > 0 && q2 == nullptr) || window < 0 || keep < 0)
    return hipErrorInvalidValue;
#define CALL(TT)                                                                              \
  {                                                                                           \
    RowAttnArgs<TT> a{(const TT*)q1, q1r, q1h, D1, (const TT*)q2, q2r, q2h, D2,               \
                      (const TT*)kc, krow, (const TT*)vc, vrow, Dv, (TT*)out, our, ouh,       \
                      tables, maxb, row_seg, positions, H, G, HB, bs, scale, softcap, tcoef,  \
                      tevery, r1, r2, talk, sink, slopes, window, keep, (const TT*)gate,      \
                      gater, sigb, vdiv, nsplit, ws_ml, ws_o};                                \
    return launch_row_attn<TT>(a, T, st);                                                     \
  }
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
