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

template <typename TY, typename TO>
__global__ void __launch_bounds__(kThreads)
layer_norm_kernel(float* __restrict__ x, const TY* __restrict__ y, float mult,
                  const float* __restrict__ w, TO* __restrict__ out, int W, float eps) {
  extern __shared__ float s_row[];
  __shared__ float s_red[kThreads / 64];
  const long long base = (long long)blockIdx.x * W;
  float sum = 0.f;
  for (int c = threadIdx.x; c < W; c += kThreads) {
    float v = x[base + c];
    if (y != nullptr) {
      v += mult * to_f32(y[base + c]);
      x[base + c] = v;
    }
    s_row[c] = v;
    sum += v;
  }
  if (w == nullptr) return;
  const float mean = block_sum<kThreads>(sum, s_red) / (float)W;
  float sq = 0.f;
  for (int c = threadIdx.x; c < W; c += kThreads) {       // a thread re-reads its own entries
    const float d = s_row[c] - mean;
    sq += d * d;
  }
  const float inv = 1.f / sqrtf(block_sum<kThreads>(sq, s_red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += kThreads)
    out[base + c] = from_f32<TO>((s_row[c] - mean) * inv * w[c]);
}

template <typename T>
__global__ void embed_pos_kernel(const T* __restrict__ table, const T* __restrict__ pos_table,
                                 const long long* __restrict__ tokens,
                                 const int* __restrict__ positions, float* __restrict__ out,
                                 long long n, int W, int V, int P) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const long long t = i / W;
    const int c = (int)(i % W);
    // the host bounds both indices; a stray one reads the table's edge instead of faulting
    const long long tok = min(max(tokens[t], 0ll), (long long)V - 1);
    const int p = min(max(positions[t], 0), P - 1);
    out[i] = to_f32(table[tok * W + c]) + to_f32(pos_table[(long long)p * W + c]);
  }
}

inline int grid_for(long long n, int block = 256) {
  const long long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : g > 65535 ? 65535 : g);
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
#define CALL_O(TO)                                                                              \
  {                                                                                             \
    if (dt_y == kF32)                                                                           \
      layer_norm_kernel<float, TO><<<rows, kThreads, lds, st>>>(x, (const float*)y, mult, w,    \
                                                                (TO*)out, W, eps);              \
    else if (dt_y == kBF16)                                                                     \
      layer_norm_kernel<bf16, TO><<<rows, kThreads, lds, st>>>(x, (const bf16*)y, mult, w,      \
                                                               (TO*)out, W, eps);               \
    else if (dt_y == kF16)                                                                      \
      layer_norm_kernel<fp16, TO><<<rows, kThreads, lds, st>>>(x, (const fp16*)y, mult, w,      \
                                                               (TO*)out, W, eps);               \
    else return hipErrorInvalidValue;                                                           \
    break;                                                                                      \
  }
  switch (dt_out) {
    case kF32: CALL_O(float)
    case kF16: CALL_O(fp16)
    case kBF16: CALL_O(bf16)
    default: return hipErrorInvalidValue;
  }
#undef CALL_O
  return hipGetLastError();
}

hipError_t sm_embed_pos(int dt, const void* table, const void* pos_table, const long long* tokens,
                        const int* positions, float* out, int T, int W, int V, int P,
                        hipStream_t st) {
  const long long n = (long long)T * W;
  if (n == 0) return hipSuccess;
  if (V < 1 || P < 1) return hipErrorInvalidValue;
#define CALL(TT) embed_pos_kernel<TT><<<grid_for(n), 256, 0, st>>>((const TT*)table, (const TT*)pos_table, tokens, positions, out, n, W, V, P)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
