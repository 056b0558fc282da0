// Layer norm with a weight and no shift, fused with what surrounds it, and the start of a
// residual stream with learned positions:
//   sm_layer_norm  the fp32 residual row takes a sublayer's output times a constant in place,
//                  x += mult * y (y in the model dtype; optional), and the same workgroup stores
//                  LN(x) * w = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w rounded to the
//                  output dtype (optional: without w only the stream moves on).
//   sm_embed_pos   x[t] = table[token[t]] + pos_table[position[t]], summed in fp32.
// One workgroup of four waves per row.  The new row is kept in LDS between the passes (sum,
// squared deviations from the mean, output), so the stream is read and written once and the
// variance is the two-pass one: no cancellation of E[x^2] - mean^2.  The partial sums of the four
// waves are added in a fixed order.  Sums, roots and products are fp32.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kThreads = 256;

// VEC: four consecutive entries per thread and step (16 bytes of fp32, 8 bytes of a 16-bit type);
// the launcher picks it when W is a multiple of 4 and the pointers are aligned for it
template <typename TY, typename TO, bool VEC>
__global__ void __launch_bounds__(kThreads)
layer_norm_kernel(float* __restrict__ x, const TY* __restrict__ y, float mult,
                  const float* __restrict__ w, TO* __restrict__ out, int W, float eps) {
  extern __shared__ float s_row[];
  __shared__ float s_red[kThreads / 64];
  constexpr int V = VEC ? 4 : 1;
  const long long base = (long long)blockIdx.x * W;
  float sum = 0.f;
  for (int c = threadIdx.x * V; c < W; c += kThreads * V) {
    if constexpr (VEC) {
      float v[4];
      load4<float>(x + base + c, v);
      if (y != nullptr) {
        float yv[4];
        load4<TY>(y + base + c, yv);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += mult * yv[e];
        store4<float>(x + base + c, v);
      }
      store4<float>(s_row + c, v);
      sum += (v[0] + v[1]) + (v[2] + v[3]);
    } else {
      float v = x[base + c];
      if (y != nullptr) {
        v += mult * to_f32(y[base + c]);
        x[base + c] = v;
      }
      s_row[c] = v;
      sum += v;
    }
  }
  if (w == nullptr) return;
  const float mean = block_sum<kThreads>(sum, s_red) / (float)W;
  float sq = 0.f;
  for (int c = threadIdx.x * V; c < W; c += kThreads * V) {   // a thread re-reads its own entries
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float d = s_row[c + e] - mean;
      sq += d * d;
    }
  }
  const float inv = 1.f / sqrtf(block_sum<kThreads>(sq, s_red) / (float)W + eps);
  for (int c = threadIdx.x * V; c < W; c += kThreads * V) {
    if constexpr (VEC) {
      float v[4], ww[4];
      load4<float>(s_row + c, v);
      load4<float>(w + c, ww);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (v[e] - mean) * inv * ww[e];
      store4<TO>(out + base + c, v);
    } else {
      out[base + c] = from_f32<TO>((s_row[c] - mean) * inv * w[c]);
    }
  }
}

// one workgroup per row; 8 entries per thread and step when W is a multiple of 8
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
embed_pos_kernel(const T* __restrict__ table, const T* __restrict__ pos_table,
                 const long long* __restrict__ tokens, const int* __restrict__ positions,
                 float* __restrict__ out, int Tn, int W, int V, int P) {
  for (int t = blockIdx.x; t < Tn; t += gridDim.x) {
    // the host bounds both indices; a stray one reads the table's edge instead of faulting
    const long long tok = min(max(tokens[t], 0ll), (long long)V - 1);
    const int p = min(max(positions[t], 0), P - 1);
    const T* a = table + tok * W;
    const T* b = pos_table + (long long)p * W;
    float* o = out + (long long)t * W;
    if constexpr (VEC) {
      for (int c = 8 * threadIdx.x; c < W; c += 8 * 256) {
        float u[8], v[8];
        load8<T>(a + c, u);
        load8<T>(b + c, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] += v[e];
        store8<float>(o + c, u);
      }
    } else {
      for (int c = threadIdx.x; c < W; c += 256) o[c] = to_f32(a[c]) + to_f32(b[c]);
    }
  }
}

}  // namespace

extern "C" {

// x fp32 [rows, W] contiguous (updated in place when y is given); y (nullable) [rows, W] in dtype
// dt_y; w (nullable) fp32 [W]; out (with w) [rows, W] in dtype dt_out.  W * 4 bytes of LDS.
hipError_t sm_layer_norm(int dt_y, int dt_out, float* x, const void* y, float mult,
                         const float* w, void* out, int rows, int W, float eps, hipStream_t st) {
  if (rows == 0 || (!y && !w)) return hipSuccess;
  if (W < 1 || (size_t)W * sizeof(float) > 65536 - 64 || (w && !out)) return hipErrorInvalidValue;
  const size_t lds = (size_t)W * sizeof(float);
  const bool vec = W % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0 &&
                   (uintptr_t)w % 16 == 0 && (uintptr_t)out % 16 == 0;
#define CALL_Y(TY, TO)                                                                          \
  {                                                                                             \
    if (vec)                                                                                    \
      layer_norm_kernel<TY, TO, true><<<rows, kThreads, lds, st>>>(x, (const TY*)y, mult, w,    \
                                                                   (TO*)out, W, eps);           \
    else                                                                                        \
      layer_norm_kernel<TY, TO, false><<<rows, kThreads, lds, st>>>(x, (const TY*)y, mult, w,   \
                                                                    (TO*)out, W, eps);          \
  }
#define CALL_O(TO)                                    \
  {                                                   \
    if (dt_y == kF32) CALL_Y(float, TO)               \
    else if (dt_y == kBF16) CALL_Y(bf16, TO)          \
    else if (dt_y == kF16) CALL_Y(fp16, TO)           \
    else return hipErrorInvalidValue;                 \
    break;                                            \
  }
  switch (dt_out) {
    case kF32: CALL_O(float)
    case kF16: CALL_O(fp16)
    case kBF16: CALL_O(bf16)
    default: return hipErrorInvalidValue;
  }
#undef CALL_O
#undef CALL_Y
  return hipGetLastError();
}

hipError_t sm_embed_pos(int dt, const void* table, const void* pos_table, const long long* tokens,
                        const int* positions, float* out, int T, int W, int V, int P,
                        hipStream_t st) {
  if ((long long)T * W == 0) return hipSuccess;
  if (V < 1 || P < 1) return hipErrorInvalidValue;
  const bool vec = W % 8 == 0 && (uintptr_t)table % 16 == 0 && (uintptr_t)pos_table % 16 == 0 &&
                   (uintptr_t)out % 16 == 0;
  const int grid = T < 65535 ? T : 65535;
#define CALL(TT)                                                                                  \
  if (vec) embed_pos_kernel<TT, true><<<grid, 256, 0, st>>>((const TT*)table, (const TT*)pos_table, \
                                                           tokens, positions, out, T, W, V, P);  \
  else embed_pos_kernel<TT, false><<<grid, 256, 0, st>>>((const TT*)table, (const TT*)pos_table,  \
                                                         tokens, positions, out, T, W, V, P)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
