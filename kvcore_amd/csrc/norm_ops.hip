// Norms that stand behind a sublayer, norms over a whole projection, and gates per head.
//
// kvc_norm_add_norm: a layer that norms a sublayer's result before it joins the stream
// (x <- x + norm_b(f(norm_a(x)))) needs, between two sublayers, the norm of the result, the sum
// into the float32 stream and the norm of the new stream: one block a row does all three with
// the row in registers (rows of a multiple of 8 values up to 16,384), or from memory otherwise.
// kvc_wide_qk_norm: the query and key norms of an attention whose norm spans all heads at once.
// kvc_latent_rows: the two latent norms of a latent attention and its one key/value row a token.
// kvc_head_gate: a sigmoid gate per head on a run of each head's columns.
// Sums of squares, scale factors and the stream are float32 whatever the storage type.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

#define S(stream) reinterpret_cast<hipStream_t>(stream)

__device__ __forceinline__ void ld8(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void ld8(const bf16_t* p, float* v) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void st8(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void st8(bf16_t* p, const float* v) {
  uint4 a;
  a.x = f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16);
  a.y = f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16);
  a.z = f32_to_bf16_bits(v[4]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[5])) << 16);
  a.w = f32_to_bf16_bits(v[6]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[7])) << 16);
  *reinterpret_cast<uint4*>(p) = a;
}

// A chunk of 8 values of a sublayer's result: the value itself, or, where the product before left
// partial sums of slices along K ([slices, T, H] float32), their sum in slice order.
template <typename TD>
__device__ __forceinline__ void ld8_sum(const TD* p, int slices, int64_t slice_stride, float* v) {
  ld8(p, v);
  for (int s = 1; s < slices; ++s) {
    float u[8];
    ld8(p + s * slice_stride, u);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] += u[i];
  }
}
template <typename TD>
__device__ __forceinline__ float ld_sum(const TD* p, int slices, int64_t slice_stride) {
  float v = to_float(p[0]);
  for (int s = 1; s < slices; ++s) v += to_float(p[s * slice_stride]);
  return v;
}

// Any width: three passes over memory, each thread rereading what it wrote itself.
template <typename TD, typename TO>
__global__ __launch_bounds__(256) void norm_add_norm_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TD* __restrict__ delta,
    const float* __restrict__ post_gain, float eps, const float* __restrict__ next_gain, float next_eps, int H,
    int slices, int64_t slice_stride) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  float* r = residual + base;
  const TD* dl = delta + base;
  float sd = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = ld_sum(dl + i, slices, slice_stride);
    sd += v * v;
  }
  const float inv_d = rsqrtf(block_sum(sd, scratch) / static_cast<float>(H) + eps);
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = r[i] + post_gain[i] * (ld_sum(dl + i, slices, slice_stride) * inv_d);
    r[i] = v;
    ss += v * v;
  }
  if (out == nullptr) return;  // the same for the whole grid
  const float inv = rsqrtf(block_sum(ss, scratch) / static_cast<float>(H) + next_eps);
  TO* o = out + base;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = from_float<TO>(next_gain[i] * (r[i] * inv));
}

// Rows of a multiple of 8 values: a thread keeps its chunks of 8 in registers, so the result and
// the stream are read once with 16- and 32-byte accesses.
template <typename TD, typename TO, int NCH>
__global__ __launch_bounds__(256) void norm_add_norm_vec_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TD* __restrict__ delta,
    const float* __restrict__ post_gain, float eps, const float* __restrict__ next_gain, float next_eps, int H,
    int slices, int64_t slice_stride) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  float d[NCH][8], v[NCH][8];
  float sd = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * 8;
    if (e < H) {
      ld8_sum(delta + base + e, slices, slice_stride, d[c]);
      ld8(residual + base + e, v[c]);
#pragma unroll
      for (int i = 0; i < 8; ++i) sd += d[c][i] * d[c][i];
    }
  }
  const float inv_d = rsqrtf(block_sum(sd, scratch) / static_cast<float>(H) + eps);
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * 8;
    if (e < H) {
      float w[8];
      ld8(post_gain + e, w);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[c][i] += w[i] * (d[c][i] * inv_d);
        ss += v[c][i] * v[c][i];
      }
      st8(residual + base + e, v[c]);
    }
  }
  if (out == nullptr) return;  // the same for the whole grid
  const float inv = rsqrtf(block_sum(ss, scratch) / static_cast<float>(H) + next_eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * 8;
    if (e < H) {
      float w[8], y[8];
      ld8(next_gain + e, w);
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = w[i] * (v[c][i] * inv);
      st8(out + base + e, y);
    }
  }
}

template <typename TD, typename TO>
void launch_norm_add_norm(TO* out, float* residual, const TD* delta, const float* post_gain, float eps,
                          const float* next_gain, float next_eps, int T, int H, int slices, hipStream_t stream) {
  const int64_t slice_stride = static_cast<int64_t>(T) * H;
  const auto misaligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) % 16) != 0; };
  const bool vec = H % 8 == 0 && H <= 8 * 2048 && !misaligned(out) && !misaligned(residual) && !misaligned(delta) &&
                   !misaligned(post_gain) && !misaligned(next_gain);
  if (vec) {
    const int nch = (H + 2047) / 2048;
#define KVC_NAN_CASE(NN)                                                                                   \
  hipLaunchKernelGGL((norm_add_norm_vec_kernel<TD, TO, NN>), dim3(T), dim3(256), 0, stream, out, residual, \
                     delta, post_gain, eps, next_gain, next_eps, H, slices, slice_stride)
    if (nch <= 1) KVC_NAN_CASE(1);
    else if (nch <= 2) KVC_NAN_CASE(2);
    else if (nch <= 4) KVC_NAN_CASE(4);
    else KVC_NAN_CASE(8);
#undef KVC_NAN_CASE
    return;
  }
  hipLaunchKernelGGL((norm_add_norm_kernel<TD, TO>), dim3(T), dim3(256), 0, stream, out, residual, delta,
                     post_gain, eps, next_gain, next_eps, H, slices, slice_stride);
}

// One block a token.  The sums of squares of the two sections first (the raw keys copied behind
// them on the way, by the thread that read them), then both scaled in place.
template <typename T>
__global__ __launch_bounds__(256) void wide_qk_norm_kernel(T* __restrict__ qkv, int64_t stride,
                                                           const float* __restrict__ q_gain,
                                                           const float* __restrict__ k_gain, float eps, int nq,
                                                           int nk, int copy_k) {
  __shared__ float scratch[16];
  T* row = qkv + static_cast<int64_t>(blockIdx.x) * stride;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const float v = to_float(row[i]);
    sq += v * v;
  }
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const T raw = row[nq + i];
    const float v = to_float(raw);
    sk += v * v;
    if (copy_k) row[nq + nk + i] = raw;
  }
  const float inv_q = rsqrtf(block_sum(sq, scratch) / static_cast<float>(nq) + eps);
  const float inv_k = rsqrtf(block_sum(sk, scratch) / static_cast<float>(nk) + eps);
  for (int i = threadIdx.x; i < nq; i += blockDim.x) row[i] = from_float<T>(q_gain[i] * (to_float(row[i]) * inv_q));
  for (int i = threadIdx.x; i < nk; i += blockDim.x)
    row[nq + i] = from_float<T>(k_gain[i] * (to_float(row[nq + i]) * inv_k));
}

// One block a token: what a latent attention makes of its down projection.  Rows of `down` hold
// [query latent of q_rank | key/value latent of rank | rot rotated key elements | ...]: the query
// latent, normed with q_gain, goes to cq; the row [rotated elements as they are | latent normed
// with kv_gain] goes to `key` and, the same values, to `value` (the one row a token that the cache
// keeps, in the place of a key and in the place of a value).
template <typename T>
__global__ __launch_bounds__(256) void latent_rows_kernel(T* __restrict__ cq, int64_t cq_stride, T* __restrict__ key,
                                                          T* __restrict__ value, int64_t kv_stride,
                                                          const T* __restrict__ down, int64_t down_stride,
                                                          const float* __restrict__ q_gain,
                                                          const float* __restrict__ kv_gain, float eps, int q_rank,
                                                          int rank, int rot) {
  __shared__ float scratch[16];
  const int64_t t = blockIdx.x;
  const T* row = down + t * down_stride;
  float sq = 0.f, sc = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = to_float(row[i]);
    sq += v * v;
  }
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = to_float(row[q_rank + i]);
    sc += v * v;
  }
  const float inv_q = rsqrtf(block_sum(sq, scratch) / static_cast<float>(q_rank) + eps);
  const float inv_c = rsqrtf(block_sum(sc, scratch) / static_cast<float>(rank) + eps);
  T* q_out = cq + t * cq_stride;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) q_out[i] = from_float<T>(q_gain[i] * (to_float(row[i]) * inv_q));
  T* k_out = key + t * kv_stride;
  T* v_out = value + t * kv_stride;
  for (int i = threadIdx.x; i < rot; i += blockDim.x) {
    const T raw = row[q_rank + rank + i];
    k_out[i] = raw;
    v_out[i] = raw;
  }
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const T c = from_float<T>(kv_gain[i] * (to_float(row[q_rank + i]) * inv_c));
    k_out[rot + i] = c;
    v_out[rot + i] = c;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
                                                        const T* __restrict__ gate, int64_t gate_stride,
                                                        int64_t total, int heads, int head_stride, int skip, int n) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t th = idx / n;
  const int e = static_cast<int>(idx - th * n);
  const int64_t t = th / heads;
  const int h = static_cast<int>(th - t * heads);
  const float g = 1.f / (1.f + expf(-to_float(gate[t * gate_stride + h])));
  out[idx] = from_float<T>(to_float(x[t * x_stride + static_cast<int64_t>(h) * head_stride + skip + e]) * g);
}

// Two softmax maps a head over the same values: rows of attn are [heads][2][dv]; the second map is
// taken off the first lambda times, the difference divided by its root mean square over the
// head's dv values (eps inside the root, no gain) and multiplied by post.  A wave a (token, head).
template <typename T, typename TA>
__global__ __launch_bounds__(256) void diff_heads_norm_kernel(T* __restrict__ out, const TA* __restrict__ attn,
                                                              int64_t attn_stride, float lambda, float eps,
                                                              float post, int64_t pairs, int heads, int dv) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t th = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (th >= pairs) return;  // the whole wave
  const int64_t t = th / heads;
  const int h = static_cast<int>(th - t * heads);
  const TA* a1 = attn + t * attn_stride + static_cast<int64_t>(2 * h) * dv;
  const TA* a2 = a1 + dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += kWave) {
    const float o = to_float(a1[e]) - lambda * to_float(a2[e]);
    ss += o * o;
  }
  const float inv = rsqrtf(wave_sum(ss) / static_cast<float>(dv) + eps) * post;
  T* o_row = out + th * dv;
  for (int e = lane; e < dv; e += kWave) o_row[e] = from_float<T>((to_float(a1[e]) - lambda * to_float(a2[e])) * inv);
}

}  // namespace

extern "C" int kvc_norm_add_norm(void* out, int out_dtype, float* residual, const void* delta, int delta_dtype,
                                 const float* post_gain, float eps, const float* next_gain, float next_eps,
                                 int T, int H, int slices, kvc_stream stream) {
  if (T < 0 || H <= 0 || slices < 1) return kvc_fail("kvc_norm_add_norm: bad sizes");
  if (slices > 1 && delta_dtype != 0) return kvc_fail("kvc_norm_add_norm: partial sums are float32");
  if (residual == nullptr || delta == nullptr || post_gain == nullptr) return kvc_fail("kvc_norm_add_norm: null operand");
  if (out != nullptr && next_gain == nullptr) return kvc_fail("kvc_norm_add_norm: the second norm needs its gain");
  if (T == 0) return 0;
  if (out == nullptr) next_gain = post_gain;  // never read
#define KVC_NAN(TD, TO)                                                                                         \
  launch_norm_add_norm<TD, TO>(static_cast<TO*>(out), residual, static_cast<const TD*>(delta), post_gain, eps, \
                               next_gain, next_eps, T, H, slices, S(stream))
  if (delta_dtype == 0 && out_dtype == 0) {
    KVC_NAN(float, float);
  } else if (delta_dtype == 0 && out_dtype == 1) {
    KVC_NAN(float, bf16_t);
  } else if (delta_dtype == 1 && out_dtype == 1) {
    KVC_NAN(bf16_t, bf16_t);
  } else if (delta_dtype == 1 && out_dtype == 0) {
    KVC_NAN(bf16_t, float);
  } else {
    return kvc_fail("kvc_norm_add_norm: unknown dtype code");
  }
#undef KVC_NAN
  return kvc_check_launch("kvc_norm_add_norm");
}

extern "C" int kvc_wide_qk_norm(void* qkv, int64_t stride, const float* q_gain, const float* k_gain, float eps,
                                int T, int nq, int nk, int copy_k, int dtype, kvc_stream stream) {
  if (T < 0 || nq <= 0 || nk <= 0 || stride < static_cast<int64_t>(nq) + nk + (copy_k ? nk : 0))
    return kvc_fail("kvc_wide_qk_norm: rows too short for the sections");
  if (q_gain == nullptr || k_gain == nullptr) return kvc_fail("kvc_wide_qk_norm: the gains are missing");
  if (T == 0) return 0;
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(wide_qk_norm_kernel<Tp>, dim3(T), dim3(256), 0, S(stream),
                                        static_cast<Tp*>(qkv), stride, q_gain, k_gain, eps, nq, nk, copy_k));
  return kvc_check_launch("kvc_wide_qk_norm");
}

extern "C" int kvc_latent_rows(void* cq, int64_t cq_stride, void* key, void* value, int64_t kv_stride,
                               const void* down, int64_t down_stride, const float* q_gain, const float* kv_gain,
                               float eps, int T, int q_rank, int rank, int rot, int dtype, kvc_stream stream) {
  if (T < 0 || q_rank < 0 || rank <= 0 || rot < 0 || cq_stride < q_rank || kv_stride < rank + rot ||
      down_stride < static_cast<int64_t>(q_rank) + rank + rot)
    return kvc_fail("kvc_latent_rows: rows too short for the sections");
  if (key == nullptr || value == nullptr || down == nullptr || kv_gain == nullptr ||
      (q_rank > 0 && (cq == nullptr || q_gain == nullptr)))
    return kvc_fail("kvc_latent_rows: null operand");
  if (T == 0) return 0;
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(latent_rows_kernel<Tp>, dim3(T), dim3(256), 0, S(stream), static_cast<Tp*>(cq),
                                        cq_stride, static_cast<Tp*>(key), static_cast<Tp*>(value), kv_stride,
                                        static_cast<const Tp*>(down), down_stride, q_gain, kv_gain, eps, q_rank, rank,
                                        rot));
  return kvc_check_launch("kvc_latent_rows");
}

extern "C" int kvc_head_gate(void* out, const void* x, int64_t x_stride, const void* gate, int64_t gate_stride,
                             int T, int heads, int head_stride, int skip, int n, int dtype, kvc_stream stream) {
  if (T < 0 || heads <= 0 || n <= 0 || skip < 0 || head_stride < skip + n ||
      x_stride < static_cast<int64_t>(heads) * head_stride || gate_stride < heads)
    return kvc_fail("kvc_head_gate: bad sizes");
  if (T == 0) return 0;
  const int64_t total = static_cast<int64_t>(T) * heads * n;
  const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(head_gate_kernel<Tp>, dim3(blocks), dim3(256), 0, S(stream),
                                        static_cast<Tp*>(out), static_cast<const Tp*>(x), x_stride,
                                        static_cast<const Tp*>(gate), gate_stride,
                                        total, heads, head_stride, skip, n));
  return kvc_check_launch("kvc_head_gate");
}

extern "C" int kvc_diff_heads_norm(void* out, const void* attn, int64_t attn_stride, int attn_dtype, float lambda,
                                   float eps, float post, int T, int heads, int dv, int dtype, kvc_stream stream) {
  if (T < 0 || heads <= 0 || dv <= 0 || attn_stride < static_cast<int64_t>(2) * heads * dv)
    return kvc_fail("kvc_diff_heads_norm: bad sizes");
  if (out == nullptr || attn == nullptr) return kvc_fail("kvc_diff_heads_norm: null operand");
  const int64_t pairs = static_cast<int64_t>(T) * heads;
  if (pairs == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((pairs + 3) / 4);
  if (attn_dtype != dtype && attn_dtype != 0) return kvc_fail("kvc_diff_heads_norm: the maps have out's dtype or are float32");
  if (attn_dtype == 0) {
    KVC_DISPATCH_DTYPE(dtype, Tp,
                       hipLaunchKernelGGL((diff_heads_norm_kernel<Tp, float>), dim3(blocks), dim3(256), 0, S(stream),
                                          static_cast<Tp*>(out), static_cast<const float*>(attn), attn_stride, lambda,
                                          eps, post, pairs, heads, dv));
  } else {
    KVC_DISPATCH_DTYPE(dtype, Tp,
                       hipLaunchKernelGGL((diff_heads_norm_kernel<Tp, Tp>), dim3(blocks), dim3(256), 0, S(stream),
                                          static_cast<Tp*>(out), static_cast<const Tp*>(attn), attn_stride, lambda,
                                          eps, post, pairs, heads, dv));
  }
  return kvc_check_launch("kvc_diff_heads_norm");
}
