// A residual stream kept as several copies that every sublayer reads as one weighted sum and
// writes back through a small mixing matrix (hyper-connections).
//
// streams [T, C, H] float32, C copies of a token's row side by side.  kvc_hyper_step does, a block
// a token and all in float32:
//   1. with y (a sublayer's result, [T, H] of either dtype, or y_slices partial sums [y_slices, T, H]
//      in float32 that are added up in their order on the way): every copy at once from the old ones,
//        x_t <- sum_s mix[s, t] x_s + mult * out_w[t] * y          (mix null: the identity;
//                                                                    out_w null: ones)
//   2. with out: u = sum_t in_w[t] x_t (in_w null: ones), out = gain * u / sqrt(mean(u^2) + eps)
//      in the model's dtype: the rows that the next sublayer (or the head) reads.
// With C = 1 and null coefficients this is the plain pre-norm step x <- x + mult * y, then the
// norm.  The write of one sublayer and the read of the next are one pass over the copies.
// kvc_spread_streams fills all copies of every token with the same row (the embedding's).

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

#define S(stream) reinterpret_cast<hipStream_t>(stream)

constexpr int kMaxCopies = 8;

template <int V>
__device__ __forceinline__ void ldv(const float* p, float* v) {
  if constexpr (V == 4) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  } else {
    v[0] = p[0];
  }
}
template <int V>
__device__ __forceinline__ void ldv(const bf16_t* p, float* v) {
  if constexpr (V == 4) {
    const uint2 a = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(a.x << 16);
    v[1] = __uint_as_float(a.x & 0xffff0000u);
    v[2] = __uint_as_float(a.y << 16);
    v[3] = __uint_as_float(a.y & 0xffff0000u);
  } else {
    v[0] = to_float(p[0]);
  }
}
template <int V>
__device__ __forceinline__ void stv(float* p, const float* v) {
  if constexpr (V == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    p[0] = v[0];
  }
}
template <int V>
__device__ __forceinline__ void stv(bf16_t* p, const float* v) {
  if constexpr (V == 4) {
    uint2 a;
    a.x = f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16);
    a.y = f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16);
    *reinterpret_cast<uint2*>(p) = a;
  } else {
    p[0] = from_float<bf16_t>(v[0]);
  }
}

// V values of a sublayer's result: the values themselves, or, where the product before left partial
// sums of slices along K ([slices, T, H] float32), their sum in slice order.
// A bias of the product that left them (one value a column, float32 or bfloat16) joins the sum last.
struct RowBias {
  const void* data;  // null: none
  int dtype;         // 0 float32, 1 bfloat16
};

template <int V, typename TY>
__device__ __forceinline__ void ld_slices(const TY* p, int slices, int64_t slice_stride, RowBias bias, int e,
                                          float* v) {
  ldv<V>(p, v);
  for (int s = 1; s < slices; ++s) {
    float u[V];
    ldv<V>(p + s * slice_stride, u);
#pragma unroll
    for (int i = 0; i < V; ++i) v[i] += u[i];
  }
  if (bias.data != nullptr) {
    float b[V];
    if (bias.dtype == 0) ldv<V>(static_cast<const float*>(bias.data) + e, b);
    else ldv<V>(static_cast<const bf16_t*>(bias.data) + e, b);
#pragma unroll
    for (int i = 0; i < V; ++i) v[i] += b[i];
  }
}

// C: the copies the registers hold (the step's own count is `copies` <= C); V: values a thread
// takes at a time (4 where H is a multiple of 4).
template <typename TY, typename TO, int C, int V>
__global__ __launch_bounds__(256) void hyper_step_kernel(
    TO* __restrict__ out, float* __restrict__ streams, const TY* __restrict__ y, const float* __restrict__ mix,
    const float* __restrict__ out_w, float mult, const float* __restrict__ in_w, const float* __restrict__ gain,
    float eps, int H, int copies, int slices, int64_t slice_stride, RowBias bias) {
  __shared__ float scratch[16];
  __shared__ float cm[C * C], co[C], ci[C];
  if (threadIdx.x < C * C) {
    const int s = threadIdx.x / C, t = threadIdx.x % C;
    float v = (s == t) ? 1.f : 0.f;
    if (mix != nullptr && s < copies && t < copies) v = mix[s * copies + t];
    cm[threadIdx.x] = v;
  }
  if (threadIdx.x < C) {
    const int t = threadIdx.x;
    co[t] = (t < copies) ? mult * (out_w != nullptr ? out_w[t] : 1.f) : 0.f;
    ci[t] = (t < copies) ? (in_w != nullptr ? in_w[t] : 1.f) : 0.f;
  }
  __syncthreads();
  float* rows = streams + static_cast<int64_t>(blockIdx.x) * copies * H;
  const TY* yr = (y != nullptr) ? y + static_cast<int64_t>(blockIdx.x) * H : nullptr;
  float ss = 0.f;
  for (int e = threadIdx.x * V; e < H; e += 256 * V) {
    float x[C][V], n[C][V];
#pragma unroll
    for (int s = 0; s < C; ++s)
      if (s < copies) ldv<V>(rows + static_cast<int64_t>(s) * H + e, x[s]);
    if (yr != nullptr) {
      float yv[V];
      ld_slices<V>(yr + e, slices, slice_stride, bias, e, yv);
#pragma unroll
      for (int t = 0; t < C; ++t) {
        if (t < copies) {
#pragma unroll
          for (int i = 0; i < V; ++i) {
            float acc = co[t] * yv[i];
#pragma unroll
            for (int s = 0; s < C; ++s)
              if (s < copies) acc = fmaf(cm[s * C + t], x[s][i], acc);
            n[t][i] = acc;
          }
          stv<V>(rows + static_cast<int64_t>(t) * H + e, n[t]);
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < C; ++t)
#pragma unroll
        for (int i = 0; i < V; ++i) n[t][i] = (t < copies) ? x[t][i] : 0.f;
    }
    if (out != nullptr) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        float u = 0.f;
#pragma unroll
        for (int t = 0; t < C; ++t)
          if (t < copies) u = fmaf(ci[t], n[t][i], u);
        ss += u * u;
      }
    }
  }
  if (out == nullptr) return;  // the same for the whole grid
  const float inv = rsqrtf(block_sum(ss, scratch) / static_cast<float>(H) + eps);
  TO* o = out + static_cast<int64_t>(blockIdx.x) * H;
  // every thread reads back what it wrote itself and forms the same sums in the same order
  for (int e = threadIdx.x * V; e < H; e += 256 * V) {
    float u[V], g[V];
#pragma unroll
    for (int i = 0; i < V; ++i) u[i] = 0.f;
#pragma unroll
    for (int t = 0; t < C; ++t) {
      if (t < copies) {
        float xv[V];
        ldv<V>(rows + static_cast<int64_t>(t) * H + e, xv);
#pragma unroll
        for (int i = 0; i < V; ++i) u[i] = fmaf(ci[t], xv[i], u[i]);
      }
    }
    ldv<V>(gain + e, g);
#pragma unroll
    for (int i = 0; i < V; ++i) u[i] = g[i] * (u[i] * inv);
    stv<V>(o + e, u);
  }
}

// The same step for rows that a block's registers hold (H <= 256 * V * NCH): every copy and the
// sublayer's result are asked for at once, before the coefficients are looked at; the new copies
// are stored and the sublayer input u stays in registers for the norm, so memory is read and
// written once and the chain of dependent loads is one load long.  The sums are formed in the
// order of the kernel above: both give the same bits.
template <typename TY, typename TO, int C, int V, int NCH>
__global__ __launch_bounds__(256) void hyper_step_regs_kernel(
    TO* __restrict__ out, float* __restrict__ streams, const TY* __restrict__ y, const float* __restrict__ mix,
    const float* __restrict__ out_w, float mult, const float* __restrict__ in_w, const float* __restrict__ gain,
    float eps, int H, int copies, int slices, int64_t slice_stride, RowBias bias) {
  __shared__ float scratch[16];
  __shared__ float cm[C * C], co[C], ci[C];
  float* rows = streams + static_cast<int64_t>(blockIdx.x) * copies * H;
  const TY* yr = (y != nullptr) ? y + static_cast<int64_t>(blockIdx.x) * H : nullptr;
  float x[NCH][C][V], yv[NCH][V];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * V;
    if (e < H) {
#pragma unroll
      for (int s = 0; s < C; ++s)
        if (s < copies) ldv<V>(rows + static_cast<int64_t>(s) * H + e, x[c][s]);
      if (yr != nullptr) ld_slices<V>(yr + e, slices, slice_stride, bias, e, yv[c]);
    }
  }
  if (threadIdx.x < C * C) {
    const int s = threadIdx.x / C, t = threadIdx.x % C;
    float v = (s == t) ? 1.f : 0.f;
    if (mix != nullptr && s < copies && t < copies) v = mix[s * copies + t];
    cm[threadIdx.x] = v;
  }
  if (threadIdx.x < C) {
    const int t = threadIdx.x;
    co[t] = (t < copies) ? mult * (out_w != nullptr ? out_w[t] : 1.f) : 0.f;
    ci[t] = (t < copies) ? (in_w != nullptr ? in_w[t] : 1.f) : 0.f;
  }
  __syncthreads();
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * V;
    if (e < H) {
      float u[V];
#pragma unroll
      for (int i = 0; i < V; ++i) u[i] = 0.f;
      if (yr != nullptr) {
        float n[C][V];
#pragma unroll
        for (int t = 0; t < C; ++t) {
          if (t < copies) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
              float acc = co[t] * yv[c][i];
#pragma unroll
              for (int s = 0; s < C; ++s)
                if (s < copies) acc = fmaf(cm[s * C + t], x[c][s][i], acc);
              n[t][i] = acc;
            }
            stv<V>(rows + static_cast<int64_t>(t) * H + e, n[t]);
#pragma unroll
            for (int i = 0; i < V; ++i) u[i] = fmaf(ci[t], n[t][i], u[i]);
          }
        }
      } else {
#pragma unroll
        for (int t = 0; t < C; ++t)
          if (t < copies) {
#pragma unroll
            for (int i = 0; i < V; ++i) u[i] = fmaf(ci[t], x[c][t][i], u[i]);
          }
      }
#pragma unroll
      for (int i = 0; i < V; ++i) {
        ss += u[i] * u[i];
        yv[c][i] = u[i];  // kept for the norm
      }
    }
  }
  if (out == nullptr) return;  // the same for the whole grid
  const float inv = rsqrtf(block_sum(ss, scratch) / static_cast<float>(H) + eps);
  TO* o = out + static_cast<int64_t>(blockIdx.x) * H;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * V;
    if (e < H) {
      float g[V], r[V];
      ldv<V>(gain + e, g);
#pragma unroll
      for (int i = 0; i < V; ++i) r[i] = g[i] * (yv[c][i] * inv);
      stv<V>(o + e, r);
    }
  }
}

__global__ __launch_bounds__(256) void spread_streams_kernel(float* __restrict__ streams, const float* __restrict__ rows,
                                                             int H, int copies, int64_t n) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t t = idx / (static_cast<int64_t>(copies) * H);
  const int e = static_cast<int>(idx % H);
  streams[idx] = rows[t * H + e];
}

template <typename TY, typename TO>
int launch_hyper(void* out, float* streams, const void* y, const float* mix, const float* out_w, float mult,
                 const float* in_w, const float* gain, float eps, int T, int H, int copies, int slices,
                 RowBias bias, hipStream_t stream) {
  const int64_t slice_stride = static_cast<int64_t>(T) * H;
  const bool v4 = H % 4 == 0;
  const int chunks = (H + (v4 ? 1024 : 256) - 1) / (v4 ? 1024 : 256);  // of 256 threads x V values
#define KVC_HYPER(C, V)                                                                                        \
  hipLaunchKernelGGL((hyper_step_kernel<TY, TO, C, V>), dim3(T), dim3(256), 0, stream, static_cast<TO*>(out), \
                     streams, static_cast<const TY*>(y), mix, out_w, mult, in_w, gain, eps, H, copies, \
                     slices, slice_stride, bias)
#define KVC_HYPER_REGS(C, V, NCH)                                                                         \
  hipLaunchKernelGGL((hyper_step_regs_kernel<TY, TO, C, V, NCH>), dim3(T), dim3(256), 0, stream,           \
                     static_cast<TO*>(out), streams, static_cast<const TY*>(y), mix, out_w, mult, in_w, gain, \
                     eps, H, copies, slices, slice_stride, bias)
  // rows that fit the registers (up to 32 groups of V values a thread for the copies) in one pass
#define KVC_HYPER_PICK(C)                                                      \
  do {                                                                         \
    if (v4 && chunks == 1) KVC_HYPER_REGS(C, 4, 1);                            \
    else if (v4 && chunks == 2) KVC_HYPER_REGS(C, 4, 2);                       \
    else if (v4 && chunks <= 4 && C * 4 <= 32) KVC_HYPER_REGS(C, 4, 4);        \
    else if (v4 && chunks <= 8 && C * 8 <= 32) KVC_HYPER_REGS(C, 4, 8);        \
    else if (!v4 && chunks <= 4) KVC_HYPER_REGS(C, 1, 4);                      \
    else if (v4) KVC_HYPER(C, 4);                                              \
    else KVC_HYPER(C, 1);                                                      \
  } while (0)
  if (copies == 1) KVC_HYPER_PICK(1);
  else if (copies == 2) KVC_HYPER_PICK(2);
  else if (copies <= 4) KVC_HYPER_PICK(4);
  else KVC_HYPER_PICK(8);
#undef KVC_HYPER_PICK
#undef KVC_HYPER_REGS
#undef KVC_HYPER
  return kvc_check_launch("kvc_hyper_step");
}

}  // namespace

extern "C" int kvc_hyper_step(void* out, int out_dtype, float* streams, const void* y, int y_dtype, int y_slices,
                              const void* y_bias, int y_bias_dtype, const float* mix, const float* out_w, float mult, const float* in_w, const float* gain,
                              float eps, int T, int H, int copies, kvc_stream stream) {
  if (T < 0 || H <= 0 || copies < 1 || copies > kMaxCopies)
    return kvc_fail("kvc_hyper_step: bad sizes (one to eight copies of the stream)");
  if (streams == nullptr) return kvc_fail("kvc_hyper_step: null stream");
  if (y_slices < 1 || (y_slices > 1 && y_dtype != 0)) return kvc_fail("kvc_hyper_step: partial sums are float32");
  if (y_bias != nullptr && (y == nullptr || (y_bias_dtype != 0 && y_bias_dtype != 1)))
    return kvc_fail("kvc_hyper_step: a bias comes with a result and is float32 or bfloat16");
  const RowBias bias{y_bias, y_bias_dtype};
  if (out != nullptr && gain == nullptr) return kvc_fail("kvc_hyper_step: the norm needs its gain");
  if (out == nullptr && y == nullptr) return 0;  // nothing to do
  if (T == 0) return 0;
  if (out == nullptr) out_dtype = 0;
  if (y == nullptr) y_dtype = 0;
  if ((out_dtype != 0 && out_dtype != 1) || (y_dtype != 0 && y_dtype != 1))
    return kvc_fail("kvc_hyper_step: unknown dtype code");
  hipStream_t st = S(stream);
  if (y_dtype == 0 && out_dtype == 0)
    return launch_hyper<float, float>(out, streams, y, mix, out_w, mult, in_w, gain, eps, T, H, copies, y_slices, bias, st);
  if (y_dtype == 0)
    return launch_hyper<float, bf16_t>(out, streams, y, mix, out_w, mult, in_w, gain, eps, T, H, copies, y_slices, bias, st);
  if (out_dtype == 0)
    return launch_hyper<bf16_t, float>(out, streams, y, mix, out_w, mult, in_w, gain, eps, T, H, copies, y_slices, bias, st);
  return launch_hyper<bf16_t, bf16_t>(out, streams, y, mix, out_w, mult, in_w, gain, eps, T, H, copies, y_slices, bias, st);
}

extern "C" int kvc_spread_streams(float* streams, const float* rows, int T, int H, int copies, kvc_stream stream) {
  if (T < 0 || H <= 0 || copies < 1) return kvc_fail("kvc_spread_streams: bad sizes");
  const int64_t n = static_cast<int64_t>(T) * copies * H;
  if (n == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  hipLaunchKernelGGL(spread_streams_kernel, dim3(blocks), dim3(256), 0, S(stream), streams, rows, H, copies, n);
  return kvc_check_launch("kvc_spread_streams");
}
