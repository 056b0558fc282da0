// Mixture-of-experts helpers around the two stacked library GEMMs of a hybrid layer's
// feed-forward:
//   sm_route_topk  router logits [T, E] fp32 -> dense routing weights [T, E] fp32 (softmax over
//                  the row's `top` largest logits at their places, zero elsewhere).  One wave per
//                  row: each lane keeps E / 64 logits in registers, `top` rounds of a wave-wide
//                  arg-max (ties: lowest index).
//   sm_route_groups  router with a choice correction and a limit to the best groups of
//                  experts: s = sigmoid(z) (or the softmax of z over all experts; weights then
//                  optionally un-normalised), the choice ranks c = s + correction, a group of
//                  neighbouring experts ranks by the sum of its largest c, only experts of the
//                  `keep` best groups are eligible, the `top` eligible experts with the largest c
//                  get s / (sum of the chosen s + eps) * scale.  One wave per row, the row's c in
//                  LDS; every arg-max breaks ties towards the lowest index.
//   sm_gated_act   act(gate) * up over stacked [gate | up] blocks (act: SiLU, ReLU, tanh-GELU or
//                  squared ReLU), expert e's block scaled by the row's routing weight; fp32 math.
//   sm_scaled_act  act(up) over stacked up blocks of experts without a gate, scaled the same way.
//   sm_write_k     rows of the key projection into the paged key cache by slot.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kMaxPerLane = 16;   // experts <= 1024

// the gate's activation: 0 SiLU, 1 ReLU, 2 tanh-GELU, 3 squared ReLU
__device__ __forceinline__ float gate_act(float g, int act) {
  if (act == 3) {
    const float r = fmaxf(g, 0.f);
    return r * r;
  }
  return act == 0 ? silu_f(g) : act == 1 ? fmaxf(g, 0.f) : gelu_tanh_f(g);
}

// wave-wide arg-max of (value, index) pairs, ties to the lowest index; every lane gets the result
__device__ __forceinline__ void wave_argmax(float& bv, int& bi) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
}

constexpr int kNone = 0x7fffffff;

// LDS per wave: c [E] (the choice ranks; -inf once an expert is chosen or its group dropped) and
// rank [n_groups] (-inf once a group is kept)
__global__ void __launch_bounds__(256)
route_groups_kernel(const float* __restrict__ z, const float* __restrict__ corr,
                    float* __restrict__ out, int T, int E, int top, int n_groups, int keep,
                    int rank_top, float scale, float sum_eps, int softmax, int normalize) {
  extern __shared__ float s_all[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row = blockIdx.x * 4 + wv;
  if (row >= T) return;                              // whole waves leave; no block barrier below
  float* c = s_all + wv * (E + n_groups);
  float* rank = c + E;
  const float* zr = z + (long long)row * E;
  float* orow = out + (long long)row * E;
  // the scores: sigmoids, or the softmax over all experts (maximum and sum wave-wide, fp32)
  float smax = 0.f, sinv = 1.f;
  if (softmax) {
    smax = -INFINITY;
    for (int e = lane; e < E; e += 64) smax = fmaxf(smax, zr[e]);
    smax = wave_max(smax);
    float ssum = 0.f;
    for (int e = lane; e < E; e += 64) ssum += expf(zr[e] - smax);
    sinv = 1.f / wave_sum(ssum);
  }
  const auto score = [&](int e) {
    return softmax ? expf(zr[e] - smax) * sinv : sigmoid_f(zr[e]);
  };
  for (int e = lane; e < E; e += 64) {
    c[e] = score(e) + (corr != nullptr ? corr[e] : 0.f);
    orow[e] = 0.f;
  }
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  if (n_groups > 1 && keep < n_groups) {
    const int per = E / n_groups;
    // a group's rank: its `rank_top` largest c summed, one lane per group
    for (int g = lane; g < n_groups; g += 64) {
      float sum = 0.f;
      int taken[4] = {-1, -1, -1, -1};               // rank_top <= 4
      for (int r = 0; r < rank_top && r < per; ++r) {
        float bv = -INFINITY;
        int bi = -1;
        for (int k = 0; k < per; ++k) {
          bool used = false;
          for (int q = 0; q < r; ++q) used |= taken[q] == k;
          if (!used && (bi < 0 || c[g * per + k] > bv)) { bv = c[g * per + k]; bi = k; }
        }
        taken[r] = bi;
        sum += bv;
      }
      rank[g] = sum;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    for (int it = 0; it < keep; ++it) {
      float bv = -INFINITY;
      int bi = kNone;
      for (int g = lane; g < n_groups; g += 64)
        if (rank[g] > bv || (rank[g] == bv && g < bi && rank[g] != -INFINITY)) { bv = rank[g]; bi = g; }
      wave_argmax(bv, bi);
      if (bi == kNone) break;
      if (lane == 0) rank[bi] = -INFINITY;           // kept: marked by -inf
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    }
    for (int e = lane; e < E; e += 64)
      if (rank[e / per] != -INFINITY) c[e] = -INFINITY;   // its group was not kept
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  }
  float den = 0.f;
  int mine[16];                                      // top <= E <= 1024: a lane wins <= 16 rounds
  int n_mine = 0;
  for (int it = 0; it < top; ++it) {
    float bv = -INFINITY;
    int bi = kNone;
    for (int e = lane; e < E; e += 64)
      if (c[e] > bv) { bv = c[e]; bi = e; }          // ascending e: ties keep the lowest index
    wave_argmax(bv, bi);
    if (bi == kNone) break;                          // fewer than `top` eligible experts
    den += score(bi);
    if ((bi & 63) == lane) {
      c[bi] = -INFINITY;
      if (n_mine < 16) mine[n_mine++] = bi;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  }
  const float k = normalize ? scale / (den + sum_eps) : scale;
  for (int q = 0; q < n_mine; ++q) orow[mine[q]] = score(mine[q]) * k;
}

template <typename T>
__global__ void scaled_act_kernel(const T* __restrict__ u, const float* __restrict__ wts,
                                  T* __restrict__ out, int Tn, int E, int ff, int ffs, int act) {
  const int width = E * ff + ffs;
  const long long n = (long long)Tn * width;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int t = (int)(i / width), col = (int)(i % width);
    const float w = col < E * ff ? wts[(long long)t * E + col / ff] : 1.f;
    out[i] = from_f32<T>(w == 0.f ? 0.f : gate_act(to_f32(u[i]), act) * w);
  }
}

// eight outputs per thread (16-byte accesses): block sizes multiples of 8, 16-bit dtypes
template <typename T>
__global__ void __launch_bounds__(256)
scaled_act_v8(const T* __restrict__ u, const float* __restrict__ wts, T* __restrict__ out, int Tn,
              int E, int ff, int ffs, int act) {
  const int width = E * ff + ffs;
  const int col = 8 * (blockIdx.x * 256 + threadIdx.x);
  if (col >= width) return;
  const int e = col < E * ff ? col / ff : -1;
  for (int t = blockIdx.y; t < Tn; t += gridDim.y) {
    const float w = e >= 0 ? wts[(long long)t * E + e] : 1.f;
    float v[8], o[8];
    if (w == 0.f) {
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = 0.f;
    } else {
      load8<T>(u + (long long)t * width + col, v);
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = gate_act(v[j], act) * w;
    }
    store8<T>(out + (long long)t * width + col, o);
  }
}

__global__ void __launch_bounds__(256)
route_topk_kernel(const float* __restrict__ z, float* __restrict__ out, int T, int E, int top) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= T) return;
  const float* zr = z + (long long)row * E;
  float val[kMaxPerLane];
  unsigned sel = 0;
#pragma unroll
  for (int q = 0; q < kMaxPerLane; ++q) {
    const int e = lane + 64 * q;
    val[q] = e < E ? zr[e] : -INFINITY;
  }
  float m0 = 0.f, den = 0.f;
  for (int it = 0; it < top; ++it) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) {
      const int e = lane + 64 * q;
      if (e < E && !((sel >> q) & 1u) && (val[q] > bv || (val[q] == bv && e < bi))) {
        bv = val[q];
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi == 0x7fffffff) break;         // fewer than `top` finite candidates
    if (it == 0) m0 = bv;
    den += expf(bv - m0);
    if ((bi & 63) == lane) sel |= 1u << (bi >> 6);
  }
  float* orow = out + (long long)row * E;
#pragma unroll
  for (int q = 0; q < kMaxPerLane; ++q) {
    const int e = lane + 64 * q;
    if (e < E) orow[e] = ((sel >> q) & 1u) ? expf(val[q] - m0) / den : 0.f;
  }
}

template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gu, const float* __restrict__ wts,
                                 T* __restrict__ out, int Tn, int E, int ff, int ffs,
                                 int act) {
  const int in_w = E * 2 * ff + 2 * ffs, out_w = E * ff + ffs;
  const long long n = (long long)Tn * out_w;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int t = (int)(i / out_w), c = (int)(i % out_w);
    const T* row = gu + (long long)t * in_w;
    float g, u, w = 1.f;
    if (c < E * ff) {
      const int e = c / ff, q = c % ff;
      w = wts[(long long)t * E + e];
      g = to_f32(row[e * 2 * ff + q]);
      u = to_f32(row[e * 2 * ff + ff + q]);
    } else {
      const int q = c - E * ff;
      g = to_f32(row[E * 2 * ff + q]);
      u = to_f32(row[E * 2 * ff + ffs + q]);
    }
    out[i] = from_f32<T>(w == 0.f ? 0.f : gate_act(g, act) * u * w);
  }
}

// eight outputs per thread (16-byte accesses): every block size a multiple of 8, 16-bit dtypes
template <typename T>
__global__ void __launch_bounds__(256)
gated_act_v8(const T* __restrict__ gu, const float* __restrict__ wts, T* __restrict__ out, int Tn,
             int E, int ff, int ffs, int act) {
  const int in_w = E * 2 * ff + 2 * ffs, out_w = E * ff + ffs;
  const int c = 8 * (blockIdx.x * 256 + threadIdx.x);
  if (c >= out_w) return;
  int e = -1, goff, uoff;
  if (c < E * ff) {
    e = c / ff;
    goff = e * 2 * ff + (c - e * ff);
    uoff = goff + ff;
  } else {
    goff = E * 2 * ff + (c - E * ff);
    uoff = goff + ffs;
  }
  for (int t = blockIdx.y; t < Tn; t += gridDim.y) {
    const T* row = gu + (long long)t * in_w;
    const float w = e >= 0 ? wts[(long long)t * E + e] : 1.f;
    float g[8], u[8], o[8];
    if (w == 0.f) {
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = 0.f;
    } else {
      load8<T>(row + goff, g);
      load8<T>(row + uoff, u);
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = gate_act(g[j], act) * u[j] * w;
    }
    store8<T>(out + (long long)t * out_w + c, o);
  }
}

template <typename T>
__global__ void write_k_kernel(const T* __restrict__ k, long long ld, T* __restrict__ cache,
                               const long long* __restrict__ slots, int Tn, int GD) {
  const long long n = (long long)Tn * GD;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int t = (int)(i / GD), c = (int)(i % GD);
    const long long s = slots[t];
    if (s >= 0) cache[s * GD + c] = k[(long long)t * ld + c];
  }
}

inline int grid_for(long long n, int block = 256) {
  long long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace

extern "C" {

hipError_t sm_route_topk(const float* z, float* out, int T, int E, int top, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (E < 1 || E > 64 * kMaxPerLane || top < 1 || top > E) return hipErrorInvalidValue;
  route_topk_kernel<<<(T + 3) / 4, 256, 0, st>>>(z, out, T, E, top);
  return hipGetLastError();
}

// z, out [T, E] fp32; corr [E] fp32.  4 * (E + n_groups) * 4 bytes of LDS per workgroup.
hipError_t sm_route_groups(const float* z, const float* corr, float* out, int T, int E, int top,
                           int n_groups, int keep, int rank_top, float scale, float sum_eps,
                           int softmax, int normalize, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (E < 1 || E > 64 * kMaxPerLane || n_groups < 1 || E % n_groups || keep < 1 ||
      keep > n_groups || top < 1 || top > keep * (E / n_groups) || rank_top < 1 || rank_top > 4)
    return hipErrorInvalidValue;
  const size_t lds = 4 * (size_t)(E + n_groups) * sizeof(float);
  route_groups_kernel<<<(T + 3) / 4, 256, lds, st>>>(z, corr, out, T, E, top, n_groups, keep,
                                                     rank_top, scale, sum_eps, softmax, normalize);
  return hipGetLastError();
}

hipError_t sm_scaled_act(int dt, const void* u, const float* wts, void* out, int T, int E, int ff,
                         int ffs, int act, hipStream_t st) {
  const long long n = (long long)T * (E * ff + ffs);
  if (n == 0) return hipSuccess;
  if (E > 0 && wts == nullptr) return hipErrorInvalidValue;
  if (ff % 8 == 0 && ffs % 8 == 0 && (dt == kBF16 || dt == kF16)) {
    const dim3 grid(((E * ff + ffs) / 8 + 255) / 256, T < 65535 ? T : 65535);
    if (dt == kBF16)
      scaled_act_v8<bf16><<<grid, 256, 0, st>>>((const bf16*)u, wts, (bf16*)out, T, E, ff, ffs, act);
    else
      scaled_act_v8<fp16><<<grid, 256, 0, st>>>((const fp16*)u, wts, (fp16*)out, T, E, ff, ffs, act);
    return hipGetLastError();
  }
#define CALL(TT) scaled_act_kernel<TT><<<grid_for(n), 256, 0, st>>>((const TT*)u, wts, (TT*)out, T, E, ff, ffs, act)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_gated_act(int dt, const void* gu, const float* wts, void* out, int T, int E, int ff,
                        int ffs, int act, hipStream_t st) {
  const long long n = (long long)T * (E * ff + ffs);
  if (n == 0) return hipSuccess;
  if (E > 0 && wts == nullptr) return hipErrorInvalidValue;
  if (ff % 8 == 0 && ffs % 8 == 0 && (dt == kBF16 || dt == kF16)) {
    const dim3 grid(((E * ff + ffs) / 8 + 255) / 256, T < 65535 ? T : 65535);
    if (dt == kBF16)
      gated_act_v8<bf16><<<grid, 256, 0, st>>>((const bf16*)gu, wts, (bf16*)out, T, E, ff, ffs,
                                                 act);
    else
      gated_act_v8<fp16><<<grid, 256, 0, st>>>((const fp16*)gu, wts, (fp16*)out, T, E, ff, ffs,
                                                 act);
    return hipGetLastError();
  }
#define CALL(TT) gated_act_kernel<TT><<<grid_for(n), 256, 0, st>>>((const TT*)gu, wts, (TT*)out, T, E, ff, ffs, act)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_write_k(int dt, const void* k, long long ld, void* cache, const long long* slots,
                      int T, int GD, hipStream_t st) {
  if ((long long)T * GD == 0) return hipSuccess;
#define CALL(TT) write_k_kernel<TT><<<grid_for((long long)T * GD), 256, 0, st>>>((const TT*)k, ld, (TT*)cache, slots, T, GD)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
