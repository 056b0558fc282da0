// Prefill attention over paged key and value caches on the matrix cores, with a soft cap, a
// linear distance bias, a sliding window that also keeps the sequence's first keys, and a
// per-head output gate -- every one optional:
//   s(i, j) = cap * tanh(q_i . k_j * scale / cap) - slope_h * (i - j)
//   row i sees key j when j <= i and (window == 0 or i - j < window or j < keep)
//   o_i = sigmoid(gate[i, h]) * sum_j softmax_j(s(i, j)) v_j
// or, with a per-head bias `sigb`, weights that are sigmoids and are not normalised:
//   o_i = sum_j sigmoid(s(i, j) + sigb_h) v_j
// q arrives as the projection left it (already normed where the design norms it), the key cache
// [blocks][bs][G][D] holds what the scores read and the value cache [blocks][bs][G / vdiv][DV]
// what is summed: the value size may differ from the key size, and `vdiv` consecutive key heads
// may share one value head (several score maps over the same values).
//
// A workgroup of NW waves takes 32 * NW consecutive rows of ONE segment and one query head.  The
// keys the tile can see are visited 32 at a time: first the tiles of the kept keys that lie below
// the window of the tile's first row, then the tiles from that window's start to the last row's
// position; what lies between is never loaded, so a long prompt's portion costs rows x (window +
// keep) and not rows x position.  A key tile is staged in LDS from the key cache (row-major, the
// score operand) and from the value cache (transposed, the value operand) and shared by the
// waves; the next tile's loads are issued before this tile's products.  Per wave (32 queries)
// and key tile, with v_mfma_f32_32x32x16:
//   S^T = K Q^T      keys on the accumulator rows, queries on the columns (lane & 31): a lane
//                    owns ONE query, so its running max / sum / correction are plain scalars;
//   O^T += V^T P^T   the accumulator registers 8s .. 8s+7 of S^T are keys {16s + 4hi + 0..3,
//                    16s + 8 + 4hi + 0..3}: exactly one k = 16 operand when the transposed value
//                    image is read in that order, so P goes from registers to the next product
//                    without touching LDS.  P is split into a 16-bit head and a 16-bit remainder
//                    (two products), which keeps ~16 mantissa bits of the fp32 weights.
// Accumulator layout of the 32x32 products: lane l, register 4j + i = row 8j + 4(l >> 5) + i,
// column l & 31; operand lanes hold k = 8(l >> 5) + 0..7.  Scores, cap, bias, softmax and the
// gate's sigmoid are fp32; the kernel serves 16-bit dtypes (fp32 models take the row kernel).
#include "seqmix.h"

using namespace lumen;

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8v __attribute__((ext_vector_type(8)));

template <typename T> struct Mma32;
template <> struct Mma32<bf16> {
  static __device__ __forceinline__ f32x16 run(uint4 a, uint4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8v, a),
                                                   __builtin_bit_cast(bf16x8v, b), c, 0, 0, 0);
  }
};
template <> struct Mma32<fp16> {
  static __device__ __forceinline__ f32x16 run(uint4 a, uint4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8v, a),
                                                  __builtin_bit_cast(f16x8v, b), c, 0, 0, 0);
  }
};

// the two halves of a packed 16-bit pair as fp32 (bf16: a shift and a mask)
template <typename T> __device__ __forceinline__ void unpack2(unsigned v, float& a, float& b);
template <> __device__ __forceinline__ void unpack2<bf16>(unsigned v, float& a, float& b) {
  a = __uint_as_float(v << 16);
  b = __uint_as_float(v & 0xffff0000u);
}
template <> __device__ __forceinline__ void unpack2<fp16>(unsigned v, float& a, float& b) {
  const lumen_f16x2 h = __builtin_bit_cast(lumen_f16x2, v);
  a = static_cast<float>(h[0]);
  b = static_cast<float>(h[1]);
}

// tanh through one exponential: 1 - 2 / (1 + e^(2x)); exact limits at both ends
__device__ __forceinline__ float tanh_exp(float x) { return 1.f - 2.f / (1.f + __expf(2.f * x)); }

template <typename T>
struct WinTileArgs {
  const T* q; long long ldq;                 // rows [T][>= H * D]
  const T* kc; const T* vc;                  // [blocks][bs][G][D], [blocks][bs][G / vdiv][DV]
  T* out;                                    // [T][H][DV]
  const T* gate; long long gater;            // gate logits [T][H], row stride (nullable)
  const int* tables; int maxb;
  const int* tiles; const int* cu; const int* start;
  int H, G, bs;
  float scale, softcap;
  const float* slopes;                       // [H] (nullable)
  int window, keep;
  const float* sigb; int vdiv;               // sigmoid weights' bias [H] (nullable); key heads per value head
};

template <typename T, int D, int DV, int NW>
__global__ void __launch_bounds__(64 * NW)
    __attribute__((amdgpu_waves_per_eu((D <= 128 && DV <= 128) ? 2 : 1)))
win_tile_attn_kernel(const WinTileArgs<T> a) {
  constexpr int QT = 32 * NW, LK = D + 8, LT = 40, NV = D / 8, NVV = DV / 8;
  __shared__ __align__(16) T s_k[32 * LK];    // key tile, row-major
  __shared__ __align__(16) T s_t[DV * LT];    // value tile, transposed [d][key]
  constexpr int kTbl = 512;                   // block-table entries of the window's keys, in LDS
  __shared__ int s_tbl[kTbl];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c = lane & 31, hi = lane >> 5;
  const int hd = blockIdx.y, g = hd / (a.H / a.G);
  const int Gv = a.G / a.vdiv, gv = g / a.vdiv;
  const float sbias = a.sigb != nullptr ? a.sigb[hd] : 0.f;
  // tiles are listed in row order, so later tiles see more keys: issue them first
  const int tix = gridDim.x - 1 - blockIdx.x;
  const int sg = a.tiles[2 * tix], row0 = a.tiles[2 * tix + 1];
  const int seg_r0 = a.cu[sg], p0 = a.start[sg];
  const int nrows = min(QT, a.cu[sg + 1] - row0);
  const int* tbl = a.tables + (long long)sg * a.maxb;
  const int window = a.window, keep = window > 0 ? a.keep : 0, bs = a.bs;

  const bool qv = 32 * w + c < nrows;
  const int qrow = row0 + 32 * w + c;
  const int pos = qv ? p0 + (qrow - seg_r0) : -1;
  uint4 qreg[D / 16];
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk)
    qreg[kk] = qv ? *reinterpret_cast<const uint4*>(a.q + (long long)qrow * a.ldq + hd * D + 16 * kk + 8 * hi)
                  : make_uint4(0, 0, 0, 0);
  const float slope = a.slopes != nullptr ? a.slopes[hd] : 0.f;
  const float cap = a.softcap, rcap = cap > 0.f ? 1.f / cap : 0.f;

  // key tiles: [0, khead) in steps of 32 (kept keys below the window), then from kwin on
  const int pos_first = p0 + (row0 - seg_r0), kend = pos_first + nrows - 1;
  const int wlo = window > 0 ? max(0, pos_first - window + 1) : 0;
  const int kwin = wlo / 32 * 32;
  const int khead = min((min(keep, wlo) + 31) / 32 * 32, kwin);
  const int kfirst = khead > 0 ? 0 : kwin;
  auto next_tile = [&](int k0) {
    const int n = k0 + 32;
    return (n >= khead && n < kwin) ? kwin : n;
  };
  const bool wave_on = 32 * w < nrows;
  const int wpos_min = pos_first + 32 * w, wpos_max = min(kend, wpos_min + 31);

  // block ids of the window's keys, so that a key's address never waits for a table load (the
  // few kept keys' entries, and entries beyond kTbl, are read from global memory)
  const int b_first = kwin / bs, b_count = kend / bs - b_first + 1;
  for (int i = tid; i < min(b_count, kTbl); i += 64 * NW) s_tbl[i] = tbl[b_first + i];
  const int bshift = (bs & (bs - 1)) == 0 ? __ffs(bs) - 1 : -1;
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  f32x16 O[DV / 32];
#pragma unroll
  for (int db = 0; db < DV / 32; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) O[db][r] = 0.f;

  // staging: one item = 4 consecutive keys x 8 channels of the key cache AND of the value cache
  // (four 16-byte loads each); the row-major image takes the keys as they are, the transposed
  // image takes eight 8-byte stores of 4 values each (transposed in registers)
  constexpr int NT = 64 * NW, ITEMS = (D + NT - 1) / NT, ITEMS_V = (DV + NT - 1) / NT;
  uint4 pk[ITEMS][4], pv[ITEMS_V][4];
  auto cache_row = [&](int j) -> long long {
    const int jb = bshift >= 0 ? j >> bshift : j / bs, jo = j - jb * bs;
    const int bi = jb - b_first;
    const int blk = (bi >= 0 && bi < kTbl) ? s_tbl[bi] : tbl[jb];
    return (long long)blk * bs + jo;
  };
  auto prefetch = [&](int k0) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int item = tid + it * NT;
      if (item < D) {
        const int kq = item / NV, part = item % NV;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const int j = k0 + 4 * kq + x;
          pk[it][x] = make_uint4(0, 0, 0, 0);
          if (j <= kend)
            pk[it][x] = *reinterpret_cast<const uint4*>(a.kc + (cache_row(j) * a.G + g) * D + 8 * part);
        }
      }
    }
#pragma unroll
    for (int it = 0; it < ITEMS_V; ++it) {
      const int item = tid + it * NT;
      if (item < DV) {
        const int kq = item / NVV, part = item % NVV;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const int j = k0 + 4 * kq + x;
          pv[it][x] = make_uint4(0, 0, 0, 0);
          if (j <= kend)
            pv[it][x] = *reinterpret_cast<const uint4*>(a.vc + (cache_row(j) * Gv + gv) * DV + 8 * part);
        }
      }
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int item = tid + it * NT;
      if (item < D) {
        const int kq = item / NV, part = item % NV;
#pragma unroll
        for (int x = 0; x < 4; ++x)
          *reinterpret_cast<uint4*>(&s_k[(4 * kq + x) * LK + 8 * part]) = pk[it][x];
      }
    }
#pragma unroll
    for (int it = 0; it < ITEMS_V; ++it) {
      const int item = tid + it * NT;
      if (item < DV) {
        const int kq = item / NVV, part = item % NVV;
        const unsigned w0[4] = {pv[it][0].x, pv[it][0].y, pv[it][0].z, pv[it][0].w};
        const unsigned w1[4] = {pv[it][1].x, pv[it][1].y, pv[it][1].z, pv[it][1].w};
        const unsigned w2[4] = {pv[it][2].x, pv[it][2].y, pv[it][2].z, pv[it][2].w};
        const unsigned w3[4] = {pv[it][3].x, pv[it][3].y, pv[it][3].z, pv[it][3].w};
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {     // word mm holds channels 2mm (low half), 2mm + 1
          // the key quads of a row are permuted by the row's group of 8 (all rows a lane
          // writes share it): lanes that differ in `part` land in different banks
          T* t0 = &s_t[(8 * part + 2 * mm) * LT + 4 * (kq ^ (part & 7))];
          *reinterpret_cast<uint2*>(t0) = make_uint2((w0[mm] & 0xffffu) | (w1[mm] << 16),
                                                     (w2[mm] & 0xffffu) | (w3[mm] << 16));
          *reinterpret_cast<uint2*>(t0 + LT) = make_uint2(
              (w0[mm] >> 16) | (w1[mm] & 0xffff0000u), (w2[mm] >> 16) | (w3[mm] & 0xffff0000u));
        }
      }
    }
  };

  prefetch(kfirst);
  for (int k0 = kfirst; k0 <= kend; k0 = next_tile(k0)) {
    __syncthreads();                       // the previous tile has been consumed
    commit();
    __syncthreads();
    const int kn = next_tile(k0);
    if (kn <= kend) prefetch(kn);
    // nothing this wave may see: past its last row, or before its first row's window and not kept
    if (!wave_on || k0 > wpos_max || (window > 0 && k0 + 31 < wpos_min - window + 1 && k0 >= keep))
      continue;

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
      const uint4 av = *reinterpret_cast<const uint4*>(&s_k[c * LK + 16 * kk + 8 * hi]);
      acc = Mma32<T>::run(av, qreg[kk], acc);
    }
    // a tile every query of the wave sees whole needs no mask
    const bool whole = k0 + 31 <= wpos_min && 32 * w + 31 < nrows &&
                       (window <= 0 || k0 >= wpos_max - window + 1 || k0 + 31 < keep);
    float sc[16];
    float mloc = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = k0 + 8 * (r >> 2) + 4 * hi + (r & 3);
      float sv = acc[r] * a.scale;
      if (cap > 0.f) sv = cap * tanh_exp(sv * rcap);
      sc[r] = sv - slope * (float)(pos - j);
    }
    if (!whole) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = k0 + 8 * (r >> 2) + 4 * hi + (r & 3);
        const bool seen = j <= pos && (window <= 0 || pos - j < window || j < keep);
        sc[r] = seen ? sc[r] : -INFINITY;
      }
    }
    if (a.sigb != nullptr) {
      // weights as they are: a hidden key's -inf gives 1 / (1 + e^inf) = 0
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = 1.f / (1.f + __expf(-(sc[r] + sbias)));
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, sc[r]);
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
      const float mn = fmaxf(m, mloc);
      const float ms = mn == -INFINITY ? 0.f : mn;
      // (v_exp_f32: this kernel serves 16-bit dtypes only, the weights are rounded to ~16 bits)
      const float corr = __expf(m - ms);
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) { sc[r] = __expf(sc[r] - ms); psum += sc[r]; }
      psum += __shfl_xor(psum, 32, 64);
      l = l * corr + psum;
      m = mn;
      if (__any(corr != 1.f)) {            // the running max moved for some query of the wave
#pragma unroll
        for (int db = 0; db < DV / 32; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) O[db][r] *= corr;
      }
    }
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      unsigned ph[4], pl[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const float a0 = sc[8 * s2 + 2 * x], a1 = sc[8 * s2 + 2 * x + 1];
        ph[x] = pk2<T>(a0, a1);                      // one packed conversion
        float h0, h1;
        unpack2<T>(ph[x], h0, h1);
        pl[x] = pk2<T>(a0 - h0, a1 - h1);
      }
      const uint4 bh = make_uint4(ph[0], ph[1], ph[2], ph[3]);
      const uint4 bl = make_uint4(pl[0], pl[1], pl[2], pl[3]);
#pragma unroll
      for (int db = 0; db < DV / 32; ++db) {
        const int row = 32 * db + c, sw = (row >> 3) & 7;     // undo the store's permutation
        const T* tp = &s_t[row * LT];
        const uint2 a0 = *reinterpret_cast<const uint2*>(tp + 4 * ((4 * s2 + hi) ^ sw));
        const uint2 a1 = *reinterpret_cast<const uint2*>(tp + 4 * ((4 * s2 + 2 + hi) ^ sw));
        const uint4 av = make_uint4(a0.x, a0.y, a1.x, a1.y);
        O[db] = Mma32<T>::run(av, bh, O[db]);
        O[db] = Mma32<T>::run(av, bl, O[db]);
      }
    }
  }
  if (qv) {
    float inv = a.sigb != nullptr ? 1.f : 1.f / l;   // l > 0: a row always sees its own key
    if (a.gate != nullptr) inv *= sigmoid_f(to_f32(a.gate[(long long)qrow * a.gater + hd]));
    T* op = a.out + ((long long)qrow * a.H + hd) * DV;
#pragma unroll
    for (int db = 0; db < DV / 32; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = 32 * db + 8 * j + 4 * hi;
        const unsigned x0 = pk2<T>(O[db][4 * j] * inv, O[db][4 * j + 1] * inv);
        const unsigned x1 = pk2<T>(O[db][4 * j + 2] * inv, O[db][4 * j + 3] * inv);
        *reinterpret_cast<uint2*>(op + d) = make_uint2(x0, x1);
      }
  }
}

template <typename T>
hipError_t launch_win_tiles(const WinTileArgs<T>& a, int ntiles, int D, int Dv, int tile_rows,
                            hipStream_t st) {
  const dim3 grid(ntiles, a.H);
#define GO(DD, DVV)                                                                          \
  if (tile_rows == 128) win_tile_attn_kernel<T, DD, DVV, 4><<<grid, 256, 0, st>>>(a);        \
  else win_tile_attn_kernel<T, DD, DVV, 2><<<grid, 128, 0, st>>>(a)
  switch (D * 1024 + Dv) {
    case 32 * 1024 + 32: GO(32, 32); break;
    case 64 * 1024 + 64: GO(64, 64); break;
    case 96 * 1024 + 96: GO(96, 96); break;
    case 128 * 1024 + 128: GO(128, 128); break;
    case 192 * 1024 + 192: GO(192, 192); break;
    case 256 * 1024 + 256: GO(256, 256); break;
    // values twice the key size (two score maps per head, or wide values)
    case 32 * 1024 + 64: GO(32, 64); break;
    case 48 * 1024 + 96: GO(48, 96); break;
    case 64 * 1024 + 128: GO(64, 128); break;
    case 96 * 1024 + 192: GO(96, 192); break;
    case 128 * 1024 + 256: GO(128, 256); break;
    default: return hipErrorInvalidValue;
  }
#undef GO
  return hipGetLastError();
}

}  // namespace

extern "C" {

// 1 when sm_win_attn_tiles has a kernel for this dtype / key size / value size
int sm_win_attn_tiles_ok(int dt, int D, int Dv) {
  if (dt != kBF16 && dt != kF16) return 0;
  if (Dv == D) return D == 32 || D == 64 || D == 96 || D == 128 || D == 192 || D == 256;
  return Dv == 2 * D && (D == 32 || D == 48 || D == 64 || D == 96 || D == 128);
}

// tiles: [ntiles, 2] int32 (segment, first row); every tile covers up to tile_rows (64 or 128)
// rows of its segment.  q rows [T][>= H * D] with row stride ldq (a multiple of 8, 16-byte
// aligned base); kc [blocks][bs][G][D], vc [blocks][bs][G / vdiv][Dv]; out [T][H][Dv] contiguous;
// gate (nullable) [T][H] with row stride gater; slopes (nullable) fp32 [H]; window 0: plain causal
// attention; sigb (nullable) fp32 [H]: sigmoid weights, not normalised.
hipError_t sm_win_attn_tiles(int dt, const void* q, long long ldq, const void* kc, const void* vc,
                             void* out, const void* gate, long long gater, const int* tables,
                             int maxb, const int* tiles, int ntiles, const int* cu,
                             const int* start, int H, int G, int D, int bs, float scale,
                             float softcap, const float* slopes, int window, int keep,
                             int tile_rows, int Dv, const float* sigb, int vdiv, hipStream_t st) {
  if (ntiles == 0) return hipSuccess;
  if (vdiv < 1 || G % vdiv || !sm_win_attn_tiles_ok(dt, D, Dv)) return hipErrorInvalidValue;
  if (G < 1 || H % G || bs < 1 || window < 0 || keep < 0 || (ldq % 8) != 0 ||
      (uintptr_t)q % 16 || (uintptr_t)kc % 16 || (uintptr_t)vc % 16 || (uintptr_t)out % 8)
    return hipErrorInvalidValue;
  if (tile_rows != 64 && tile_rows != 128) return hipErrorInvalidValue;
#define CALL(TT)                                                                               \
  {                                                                                            \
    WinTileArgs<TT> a{(const TT*)q, ldq, (const TT*)kc, (const TT*)vc, (TT*)out,               \
                      (const TT*)gate, gater, tables, maxb, tiles, cu, start, H, G, bs, scale, \
                      softcap, slopes, window, keep, sigb, vdiv};                              \
    return launch_win_tiles<TT>(a, ntiles, D, Dv, tile_rows, st);                              \
  }
  if (dt == kBF16) CALL(bf16)
  if (dt == kF16) CALL(fp16)
#undef CALL
  return hipErrorInvalidValue;
}

}  // extern "C"
