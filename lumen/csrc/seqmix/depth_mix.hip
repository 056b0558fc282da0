// Kernels of stacks whose layers run their sublayers in parallel on one normed input and read a
// depth-weighted average of all earlier results, and of the mixers such a stack brings along:
//
//   sm_embed_scaled   out[t] = table[token[t]] * scale in fp32 (the start of the stream)
//   sm_depth_mix      one pass per layer over a row of the stream:
//                       X_n = x + sum_k scale_k * y_k        (<= 3 sublayer outputs, per-channel
//                                                             fp32 scales), stored in the history
//                       x'  = sum_{j <= n} mix[j] * X_j      (the history is [L + 1][T][W] fp32)
//                       h   = x' / sqrt(mean(x'^2) + eps) * w, rounded to the compute dtype
//                     one workgroup per row, the new row kept in LDS between the two passes
//   sm_rotary_write   the q and k heads of a fused projection's row turned in place on their first
//                     `dims` entries (pair layout (2i, 2i+1) or half layout (i, i + dims/2)), the
//                     turned keys and the value columns copied into their paged caches
//   sm_min_gru        S_t = (1 - z_t) S_(t-1) + z_t c_t per channel over the rows of a segment,
//                     z = sigmoid(zl + b_z), c = u + shift (u >= 0) | sigmoid(u), u = xl + b_x,
//                     out = S_t * silu(gl); the fp32 state lives in [slots][width] across steps.
//                     Prompt portions are cut into chunks: pass 1 reduces every chunk to its affine
//                     map S -> A S + B, pass 2 walks the chunks' maps (few) and replays each chunk
//                     from its true start state -- a row's result is the same fp32 recurrence
//                     whichever way the step was cut, up to the rounding of A S + B.
//   sm_diff_combine   two score maps' outputs over the same values -> a1 - lam * a2, unit RMS per
//                     head, a constant, an element-wise sigmoid gate
//   sm_soft_cap       cap * tanh(z / cap) in fp32
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kThreads = 256;

template <typename T, bool VEC>
__global__ void __launch_bounds__(kThreads)
embed_scaled_kernel(const T* __restrict__ table, const long long* __restrict__ tokens,
                    float* __restrict__ out, int W, int V, float scale) {
  long long tok = tokens[blockIdx.x];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
  const T* src = table + tok * W;
  float* dst = out + (long long)blockIdx.x * W;
  if constexpr (VEC) {
    for (int c = threadIdx.x * 4; c < W; c += kThreads * 4) {
      float v[4];
      load4<T>(src + c, v);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] *= scale;
      store4<float>(dst + c, v);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += kThreads) dst[c] = to_f32(src[c]) * scale;
  }
}

template <typename TY>
struct MixArgs {
  float* hist; int n; long long plane;       // plane = T * W
  const float* x;
  const TY* y[3]; const float* sc[3];
  const float* mix; const float* w;
  float* xn;
};

template <typename TY, typename TO, bool VEC>
__global__ void __launch_bounds__(kThreads)
depth_mix_kernel(const MixArgs<TY> a, TO* __restrict__ h, int W, float eps) {
  extern __shared__ float s_row[];
  __shared__ float s_red[kThreads / 64];
  constexpr int V = VEC ? 4 : 1;
  const long long base = (long long)blockIdx.x * W;
  float* hn = a.hist + (long long)a.n * a.plane + base;
  const float mn = a.mix[a.n];
  float sq = 0.f;
  for (int c = threadIdx.x * V; c < W; c += kThreads * V) {
    float v[V], acc[V];
    if constexpr (VEC) load4<float>(a.x + base + c, v);
    else v[0] = a.x[base + c];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      if (a.y[k] == nullptr) continue;
      float yv[V], sv[V];
      if constexpr (VEC) {
        load4<TY>(a.y[k] + base + c, yv);
        load4<float>(a.sc[k] + c, sv);
      } else {
        yv[0] = to_f32(a.y[k][base + c]);
        sv[0] = a.sc[k][c];
      }
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] += yv[e] * sv[e];
    }
    if constexpr (VEC) store4<float>(hn + c, v);
    else hn[c] = v[0];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.f;
    for (int j = 0; j < a.n; ++j) {
      const float mj = a.mix[j];
      float hv[V];
      if constexpr (VEC) load4<float>(a.hist + (long long)j * a.plane + base + c, hv);
      else hv[0] = a.hist[(long long)j * a.plane + base + c];
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += mj * hv[e];
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
      acc[e] += mn * v[e];
      sq += acc[e] * acc[e];
    }
    if constexpr (VEC) {
      store4<float>(a.xn + base + c, acc);
      store4<float>(s_row + c, acc);
    } else {
      a.xn[base + c] = acc[0];
      s_row[c] = acc[0];
    }
  }
  if (a.w == nullptr) return;
  const float inv = 1.f / sqrtf(block_sum<kThreads>(sq, s_red) / (float)W + eps);
  for (int c = threadIdx.x * V; c < W; c += kThreads * V) {   // a thread re-reads its own entries
    if constexpr (VEC) {
      float v[4], ww[4];
      load4<float>(s_row + c, v);
      load4<float>(a.w + c, ww);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = v[e] * inv * ww[e];
      store4<TO>(h + base + c, v);
    } else {
      h[base + c] = from_f32<TO>(s_row[c] * inv * a.w[c]);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(kThreads)
rotary_write_kernel(T* __restrict__ z, long long ld, const int* __restrict__ positions,
                    const long long* __restrict__ slots, T* __restrict__ kcache,
                    T* __restrict__ vcache, int nq, int nk, int D, int dims,
                    const float* __restrict__ inv_freq, int half, int vw) {
  const int t = blockIdx.x;
  T* row = z + (long long)t * ld;
  const float pos = (float)positions[t];
  const int hp = dims / 2, n = nq + nk;
  for (int i = threadIdx.x; i < n * hp; i += kThreads) {
    const int hd = i / hp, pr = i % hp;
    float sn, cs;
    sincosf(pos * inv_freq[pr], &sn, &cs);
    T* p = row + hd * D;
    const int i0 = half ? pr : 2 * pr, i1 = half ? pr + hp : 2 * pr + 1;
    const float u = to_f32(p[i0]), v = to_f32(p[i1]);
    p[i0] = from_f32<T>(u * cs - v * sn);
    p[i1] = from_f32<T>(v * cs + u * sn);
  }
  if (kcache == nullptr) return;
  const long long s = slots[t];
  if (s < 0) return;
  __syncthreads();                                   // the turned keys are read back below
  const int kw = nk * D;
  const T* ks = row + nq * D;
  T* kd = kcache + s * kw;
  for (int c = threadIdx.x; c < kw; c += kThreads) kd[c] = ks[c];
  const T* vs = ks + kw;
  T* vd = vcache + s * vw;
  for (int c = threadIdx.x; c < vw; c += kThreads) vd[c] = vs[c];
}

// ---- minGRU ------------------------------------------------------------------------------------
template <typename T>
struct GruArgs {
  const T* zxg; long long ld;
  const float* bz; const float* bx;
  float* state; T* out;
  const int* cu; const int* slot; const int* start;
  int width; float shift;
  float* ab;                                 // [chunks][2][width] affine maps (chunked form)
  const int* tiles; int chunk;               // per chunk (segment, first row); rows per chunk
};

template <typename T>
__device__ __forceinline__ void gru_gates(const GruArgs<T>& a, long long r, int c, float bz,
                                          float bx, float& z, float& cand) {
  const T* p = a.zxg + r * a.ld;
  z = sigmoid_f(to_f32(p[c]) + bz);
  const float u = to_f32(p[a.width + c]) + bx;
  cand = u >= 0.f ? u + a.shift : sigmoid_f(u);
}

// one thread per (segment, channel): the whole segment in order (short segments, decode rows)
template <typename T>
__global__ void __launch_bounds__(64)
min_gru_seq_kernel(const GruArgs<T> a) {
  const int seg = blockIdx.y, c = blockIdx.x * 64 + threadIdx.x;
  if (c >= a.width) return;
  const int r0 = a.cu[seg], r1 = a.cu[seg + 1];
  if (r1 <= r0) return;
  float* sp = a.state + (long long)a.slot[seg] * a.width + c;
  float S = a.start[seg] > 0 ? *sp : 0.f;
  const float bz = a.bz[c], bx = a.bx[c];
  for (int r = r0; r < r1; ++r) {
    float z, cand;
    gru_gates(a, r, c, bz, bx, z, cand);
    S = (1.f - z) * S + z * cand;
    const float g = to_f32(a.zxg[(long long)r * a.ld + 2 * a.width + c]);
    a.out[(long long)r * a.width + c] = from_f32<T>(S * silu_f(g));
  }
  *sp = S;
}

// chunked form: a tile of `chunk` rows is cut into kSub sub-chunks (grid z), each a short serial
// walk, so that a step's prompt rows keep thousands of waves busy.
constexpr int kSub = 4;
constexpr int kGruUnroll = 8;

template <typename T>
struct GruSpan {
  int seg, ra, rb, s0, s1, q, q_first;       // rows [ra, rb) of segment rows [s0, s1); map index
  __device__ __forceinline__ GruSpan(const GruArgs<T>& a) {
    const int ch = blockIdx.y, z = blockIdx.z, sub = (a.chunk + kSub - 1) / kSub;
    seg = a.tiles[2 * ch];
    const int r0 = a.tiles[2 * ch + 1];
    s0 = a.cu[seg];
    s1 = a.cu[seg + 1];
    const int r1 = min(r0 + a.chunk, s1);
    ra = min(r0 + z * sub, r1);
    rb = min(ra + sub, r1);
    q = ch * kSub + z;
    q_first = (ch - (r0 - s0) / a.chunk) * kSub;
  }
};

// pass 1: sub-chunk -> (A, B) with S_end = A S_begin + B; rows are loaded kGruUnroll at a time
// before the serial updates, so the walk is not one memory round trip per row
template <typename T>
__global__ void __launch_bounds__(64)
min_gru_reduce_kernel(const GruArgs<T> a) {
  const int c = blockIdx.x * 64 + threadIdx.x;
  if (c >= a.width) return;
  const GruSpan<T> sp(a);
  if (sp.rb <= sp.ra) return;
  const float bz = a.bz[c], bx = a.bx[c];
  float A = 1.f, B = 0.f;
  for (int r = sp.ra; r < sp.rb; r += kGruUnroll) {
    float zl[kGruUnroll], xl[kGruUnroll];
#pragma unroll
    for (int u = 0; u < kGruUnroll; ++u) {
      const T* p = a.zxg + (long long)min(r + u, sp.rb - 1) * a.ld;
      zl[u] = to_f32(p[c]);
      xl[u] = to_f32(p[a.width + c]);
    }
#pragma unroll
    for (int u = 0; u < kGruUnroll; ++u) {
      if (r + u < sp.rb) {
        const float z = sigmoid_f(zl[u] + bz), uu = xl[u] + bx;
        const float cand = uu >= 0.f ? uu + a.shift : sigmoid_f(uu);
        A *= 1.f - z;
        B = (1.f - z) * B + z * cand;
      }
    }
  }
  a.ab[((long long)sp.q * 2) * a.width + c] = A;
  a.ab[((long long)sp.q * 2 + 1) * a.width + c] = B;
}

// pass 2: a sub-chunk's start state from the maps of those before it in its segment, then the
// sub-chunk replayed; the segment's last one parks the end state in its own map's place
template <typename T>
__global__ void __launch_bounds__(64)
min_gru_replay_kernel(const GruArgs<T> a) {
  const int c = blockIdx.x * 64 + threadIdx.x;
  if (c >= a.width) return;
  const GruSpan<T> sp(a);
  if (sp.rb <= sp.ra) return;
  float S = a.start[sp.seg] > 0 ? a.state[(long long)a.slot[sp.seg] * a.width + c] : 0.f;
  for (int k = sp.q_first; k < sp.q; ++k)
    S = a.ab[((long long)k * 2) * a.width + c] * S + a.ab[((long long)k * 2 + 1) * a.width + c];
  const float bz = a.bz[c], bx = a.bx[c];
  for (int r = sp.ra; r < sp.rb; r += kGruUnroll) {
    float zl[kGruUnroll], xl[kGruUnroll], gl[kGruUnroll];
#pragma unroll
    for (int u = 0; u < kGruUnroll; ++u) {
      const T* p = a.zxg + (long long)min(r + u, sp.rb - 1) * a.ld;
      zl[u] = to_f32(p[c]);
      xl[u] = to_f32(p[a.width + c]);
      gl[u] = to_f32(p[2 * a.width + c]);
    }
#pragma unroll
    for (int u = 0; u < kGruUnroll; ++u) {
      if (r + u < sp.rb) {
        const float z = sigmoid_f(zl[u] + bz), uu = xl[u] + bx;
        const float cand = uu >= 0.f ? uu + a.shift : sigmoid_f(uu);
        S = (1.f - z) * S + z * cand;
        a.out[(long long)(r + u) * a.width + c] = from_f32<T>(S * silu_f(gl[u]));
      }
    }
  }
  if (sp.rb == sp.s1) a.ab[((long long)sp.q * 2) * a.width + c] = S;   // stored once all have read
}

// pass 3: the parked end states into the slots (after every sub-chunk has read its start state)
template <typename T>
__global__ void __launch_bounds__(64)
min_gru_store_kernel(const GruArgs<T> a) {
  const int c = blockIdx.x * 64 + threadIdx.x;
  if (c >= a.width) return;
  const GruSpan<T> sp(a);
  if (sp.rb <= sp.ra || sp.rb != sp.s1) return;
  a.state[(long long)a.slot[sp.seg] * a.width + c] = a.ab[((long long)sp.q * 2) * a.width + c];
}

// one wave per (row, head); VEC: a lane owns 4 consecutive channels of every 256
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
diff_combine_kernel(const T* __restrict__ av, const T* __restrict__ gate, long long gater,
                    T* __restrict__ out, int Tn, int G, int rep, int Dv, float lam,
                    float out_scale, float eps) {
  const int lane = threadIdx.x & 63;
  const long long wid = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int H = G * rep;
  if (wid >= (long long)Tn * H) return;
  const long long t = wid / H;
  const int h = (int)(wid % H), g = h / rep, r = h % rep;
  const T* a1 = av + ((t * G + g) * 2 * rep + r) * Dv;
  const T* a2 = a1 + (long long)rep * Dv;
  float o[8], sq = 0.f;                               // Dv <= 512
  T* op = out + (t * H + h) * Dv;
  const T* gp = gate ? gate + t * gater + (long long)h * Dv : nullptr;
  if constexpr (VEC) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int d = 4 * lane + 256 * b;
      float x1[4] = {0.f, 0.f, 0.f, 0.f}, x2[4] = {0.f, 0.f, 0.f, 0.f};
      if (d < Dv) {
        load4<T>(a1 + d, x1);
        load4<T>(a2 + d, x2);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        o[4 * b + e] = x1[e] - lam * x2[e];
        sq += o[4 * b + e] * o[4 * b + e];
      }
    }
    const float inv = out_scale / sqrtf(wave_sum(sq) / (float)Dv + eps);
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int d = 4 * lane + 256 * b;
      if (d < Dv) {
        float gv[4] = {0.f, 0.f, 0.f, 0.f}, r[4];
        if (gp) load4<T>(gp + d, gv);
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = o[4 * b + e] * inv * (gp ? sigmoid_f(gv[e]) : 1.f);
        store4<T>(op + d, r);
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = lane + 64 * e;
      o[e] = d < Dv ? to_f32(a1[d]) - lam * to_f32(a2[d]) : 0.f;
      sq += o[e] * o[e];
    }
    const float inv = out_scale / sqrtf(wave_sum(sq) / (float)Dv + eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = lane + 64 * e;
      if (d < Dv) op[d] = from_f32<T>(o[e] * inv * (gp ? sigmoid_f(to_f32(gp[d])) : 1.f));
    }
  }
}

template <typename T>
__global__ void soft_cap_kernel(const T* __restrict__ z, float* __restrict__ out, long long n,
                                float cap) {
  const float r = 1.f / cap;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x)
    out[i] = cap * tanhf(to_f32(z[i]) * r);
}

inline int grid_for(long long n, int block = 256) {
  const long long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : g > 65535 ? 65535 : g);
}

}  // namespace

extern "C" {

hipError_t sm_embed_scaled(int dt, const void* table, const long long* tokens, float* out, int T,
                           int W, int V, float scale, hipStream_t st) {
  if (T == 0) return hipSuccess;
  const bool vec = W % 4 == 0 && (uintptr_t)table % 16 == 0 && (uintptr_t)out % 16 == 0;
#define CALL(TT)                                                                                \
  if (vec) embed_scaled_kernel<TT, true><<<T, kThreads, 0, st>>>((const TT*)table, tokens, out, \
                                                                 W, V, scale);                  \
  else embed_scaled_kernel<TT, false><<<T, kThreads, 0, st>>>((const TT*)table, tokens, out, W, \
                                                              V, scale)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_depth_mix(int dt_y, int dt_out, float* hist, int n, const float* x, const void* y0,
                        const float* s0, const void* y1, const float* s1, const void* y2,
                        const float* s2, const float* mix, const float* w, float* xn, void* h,
                        int T, int W, float eps, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (n < 1 || y0 == nullptr || (w != nullptr && h == nullptr)) return hipErrorInvalidValue;
  const size_t lds = (size_t)W * sizeof(float);
  if (lds > 65536) return hipErrorInvalidValue;
  const auto al = [](const void* p) { return (uintptr_t)p % 16 == 0; };
  const bool vec = W % 4 == 0 && al(hist) && al(x) && al(y0) && al(s0) && al(y1) && al(s1) &&
                   al(y2) && al(s2) && al(w) && al(xn) && al(h);
#define CALL_Y(TY, TO)                                                                          \
  {                                                                                             \
    MixArgs<TY> a{hist, n, (long long)T * W, x, {(const TY*)y0, (const TY*)y1, (const TY*)y2},  \
                  {s0, s1, s2}, mix, w, xn};                                                    \
    if (vec) depth_mix_kernel<TY, TO, true><<<T, kThreads, lds, st>>>(a, (TO*)h, W, eps);       \
    else depth_mix_kernel<TY, TO, false><<<T, kThreads, lds, st>>>(a, (TO*)h, W, eps);          \
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

hipError_t sm_rotary_write(int dt, void* z, long long ld, const int* positions,
                           const long long* slots, void* kcache, void* vcache, int T, int nq,
                           int nk, int D, int dims, const float* inv_freq, int half, int vw,
                           hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (dims % 2 || dims > D || dims < 0 || (kcache == nullptr && nk != 0) ||
      (kcache != nullptr && vcache == nullptr && vw != 0) || ld < (long long)(nq + nk) * D + vw)
    return hipErrorInvalidValue;
#define CALL(TT) rotary_write_kernel<TT><<<T, kThreads, 0, st>>>((TT*)z, ld, positions, slots, (TT*)kcache, (TT*)vcache, nq, nk, D, dims, inv_freq, half, vw)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

// tiles == nullptr: one thread per channel walks a whole segment (segments 0 .. n_seg - 1 of
// cu / slot / start; rows are absolute).  Else the chunked form over the n_chunks chunks listed
// in `tiles` ([n_chunks][2] = segment, first row; a segment's chunks consecutive, `chunk` rows
// each from the segment's first row on), with `ab` a scratch of n_chunks * sm_min_gru_sub() * 2 *
// width floats.
int sm_min_gru_sub() { return kSub; }

hipError_t sm_min_gru(int dt, const void* zxg, long long ld, const float* bz, const float* bx,
                      float* state, void* out, const int* cu, const int* slot, const int* start,
                      int n_seg, int width, float shift, float* ab, const int* tiles,
                      int n_chunks, int chunk, hipStream_t st) {
  if ((tiles == nullptr && n_seg == 0) || (tiles != nullptr && n_chunks == 0)) return hipSuccess;
  if (width < 1 || ld < 3ll * width) return hipErrorInvalidValue;
  const int gx = (width + 63) / 64;
#define CALL(TT)                                                                                \
  {                                                                                             \
    GruArgs<TT> a{(const TT*)zxg, ld, bz, bx, state, (TT*)out, cu, slot, start, width, shift,   \
                  ab, tiles, chunk};                                                            \
    if (tiles == nullptr) {                                                                     \
      min_gru_seq_kernel<TT><<<dim3(gx, n_seg), 64, 0, st>>>(a);                                \
    } else {                                                                                    \
      if (ab == nullptr || chunk < 1) return hipErrorInvalidValue;                              \
      min_gru_reduce_kernel<TT><<<dim3(gx, n_chunks, kSub), 64, 0, st>>>(a);                    \
      min_gru_replay_kernel<TT><<<dim3(gx, n_chunks, kSub), 64, 0, st>>>(a);                    \
      min_gru_store_kernel<TT><<<dim3(gx, n_chunks, kSub), 64, 0, st>>>(a);                     \
    }                                                                                           \
  }
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_diff_combine(int dt, const void* av, const void* gate, long long gater, void* out,
                           int T, int G, int rep, int Dv, float lam, float out_scale, float eps,
                           hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (Dv < 1 || Dv > 512 || G < 1 || rep < 1) return hipErrorInvalidValue;
  const long long waves = (long long)T * G * rep;
  const bool vec = Dv % 4 == 0 && (uintptr_t)av % 16 == 0 && (uintptr_t)out % 16 == 0 &&
                   (gate == nullptr || ((uintptr_t)gate % 16 == 0 && gater % 4 == 0));
#define CALL(TT)                                                                                \
  if (vec) diff_combine_kernel<TT, true><<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(          \
      (const TT*)av, (const TT*)gate, gater, (TT*)out, T, G, rep, Dv, lam, out_scale, eps);     \
  else diff_combine_kernel<TT, false><<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(             \
      (const TT*)av, (const TT*)gate, gater, (TT*)out, T, G, rep, Dv, lam, out_scale, eps)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_soft_cap(int dt, const void* z, float* out, long long n, float cap,
                       hipStream_t st) {
  if (n == 0) return hipSuccess;
  if (!(cap > 0.f)) return hipErrorInvalidValue;
#define CALL(TT) soft_cap_kernel<TT><<<grid_for(n), 256, 0, st>>>((const TT*)z, out, n, cap)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
