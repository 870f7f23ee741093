// Paged attention, general kernel: one 64-lane wave per (token, query head).
//
// Serves every batch shape (portions of prompts beside single decoded tokens), both
// storage types and every head size up to 512 (heads above 256 in instances of their own).  A token at
// position p reads keys first..p of its request through the block table, 64 keys a
// tile: each lane scores one key (a float32 dot product over the head in index
// order), the tile is folded into a running softmax (float32 max, sum and output
// accumulators), then the lanes split the head's elements to add p_j * V_j in key
// order.  K pages are [kv head, page_size, d], V pages [kv head, dv, page_size]: keys of d
// elements and values of dv, which need not be equal.  What a token computes depends on its position, window and cache content
// only: not on the batch it is in nor on how its request was cut into steps.  Two options:
// `slopes` (a value per query head) takes slope * (position - key position) off every score, and
// `chunk` lets a token see only the keys of its own chunk of that many positions; `sinks` (a value
// per query head) adds exp(sink) to the softmax's denominator and nothing to the weighted sum.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kMaxHeadDim = 512;    // the widest head served
constexpr int kUsualHeadDim = 256;  // heads up to this size take the instances with half the registers

template <typename T>
struct Vec16;  // 16 bytes of T
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  float4 v;
  __device__ __forceinline__ float get(int i) const { return (&v.x)[i]; }
};
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  uint4 v;
  __device__ __forceinline__ float get(int i) const {
    const uint32_t word = (&v.x)[i >> 1];
    return __uint_as_float((i & 1) ? (word & 0xffff0000u) : (word << 16));
  }
};

template <typename T, int MAXD>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void paged_attention_wave_kernel(
    T* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ table, int table_stride,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ slots, int nh, int nkv, int d, int dv, int page_size, int num_pages,
    float scale, int window, const float* __restrict__ slopes, int chunk, const float* __restrict__ sinks,
    int out_f32) {
  __shared__ float q_s[kWavesPerBlock][MAXD];
  __shared__ float p_s[kWavesPerBlock][kWave];
  __shared__ int64_t off_s[kWavesPerBlock][kWave];   // K row of each key of the tile
  __shared__ int64_t voff_s[kWavesPerBlock][kWave];  // V column of each key of the tile

  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int h_raw = blockIdx.y * kWavesPerBlock + wave;
  const bool head_live = h_raw < nh;
  const int h = head_live ? h_raw : nh - 1;
  // the results in the operands' type, or (out_f32) as the float32 sums they are
  T* o = out + (static_cast<int64_t>(t) * nh + h) * dv;
  float* o32 = reinterpret_cast<float*>(out) + (static_cast<int64_t>(t) * nh + h) * dv;

  const int req = token_req[t];
  if (req < 0) {  // padding token: the whole block takes this branch
    if (head_live)
      for (int i = lane; i < dv; i += kWave) {
        if (out_f32) o32[i] = 0.f;
        else o[i] = from_float<T>(0.f);
      }
    return;
  }
  const int pos = positions[t];
  int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // chunks are counted from the sequence's first position: a token sees its own chunk's keys
  if (chunk > 0 && (pos / chunk) * chunk > first) first = (pos / chunk) * chunk;
  const int32_t* row = table + static_cast<int64_t>(slots[req]) * table_stride;
  const int hk = h / (nh / nkv);
  const float slope = slopes != nullptr ? slopes[h] : 0.f;  // taken off the score per token of distance

  const T* qh = q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * d;
  for (int i = lane; i < d; i += kWave) q_s[wave][i] = to_float(qh[i]);
  __syncthreads();

  // a sink is one more logit in the denominator that brings no value along: the running softmax
  // starts from it instead of from nothing
  float m = -INFINITY, l = 0.f;
  if (sinks != nullptr) {
    m = sinks[h];
    l = 1.f;
  }
  float acc[MAXD / kWave];
#pragma unroll
  for (int i = 0; i < MAXD / kWave; ++i) acc[i] = 0.f;

  constexpr int VN = Vec16<T>::N;
  const int64_t head_off = static_cast<int64_t>(hk) * page_size * d;
  const int64_t page_elems = static_cast<int64_t>(nkv) * page_size * d;
  const int64_t v_head_off = static_cast<int64_t>(hk) * page_size * dv;
  const int64_t v_page_elems = static_cast<int64_t>(nkv) * page_size * dv;

  for (int tile = first; tile <= pos; tile += kWave) {
    const int key = tile + lane;
    const bool valid = key <= pos;
    float s = -INFINITY;
    int64_t off = -1, voff = -1;
    if (valid) {
      const int page = row[key / page_size];
      if (page > 0 && page < num_pages) {
        off = static_cast<int64_t>(page) * page_elems + head_off +
              static_cast<int64_t>(key % page_size) * d;
        voff = static_cast<int64_t>(page) * v_page_elems + v_head_off + key % page_size;
        const T* kr = k_cache + off;
        float dot = 0.f;
        if (d % VN == 0) {
          for (int i = 0; i < d; i += VN) {
            const Vec16<T> kv = *reinterpret_cast<const Vec16<T>*>(kr + i);
#pragma unroll
            for (int e = 0; e < VN; ++e) dot = fmaf(q_s[wave][i + e], kv.get(e), dot);
          }
        } else {  // a key size that 16-byte loads do not divide: element by element
          for (int i = 0; i < d; ++i) dot = fmaf(q_s[wave][i], to_float(kr[i]), dot);
        }
        s = dot * scale - slope * static_cast<float>(pos - key);
      }
    }
    const float tile_max = wave_max(s);
    const float m_new = fmaxf(m, tile_max);
    // a tile with no readable key (pages given back behind a window) leaves the state alone
    const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    const float tile_sum = wave_sum(p);
    l = l * alpha + tile_sum;
    m = m_new;
    __syncthreads();
    p_s[wave][lane] = p;
    off_s[wave][lane] = off;
    voff_s[wave][lane] = voff;
    __syncthreads();
    const int n_keys = (pos - tile + 1 < kWave) ? pos - tile + 1 : kWave;
#pragma unroll
    for (int i = 0; i < MAXD / kWave; ++i) acc[i] *= alpha;
    for (int j = 0; j < n_keys; ++j) {
      const int64_t vo = voff_s[wave][j];
      if (vo < 0) continue;
      const float pj = p_s[wave][j];
      const T* vr = v_cache + vo;  // element e of this key is at vr[e * page_size]
#pragma unroll
      for (int i = 0; i < MAXD / kWave; ++i) {
        const int e = lane + i * kWave;
        if (e < dv) acc[i] = fmaf(pj, to_float(vr[static_cast<int64_t>(e) * page_size]), acc[i]);
      }
    }
  }
  if (!head_live) return;
  const float inv = (l > 0.f) ? 1.f / l : 0.f;
#pragma unroll
  for (int i = 0; i < MAXD / kWave; ++i) {
    const int e = lane + i * kWave;
    if (e < dv) {
      if (out_f32) o32[e] = acc[i] * inv;
      else o[e] = from_float<T>(acc[i] * inv);
    }
  }
}

}  // namespace

extern "C" int kvc_paged_attention(void* out, const void* q, int64_t q_stride, const void* k_cache,
                                   const void* v_cache, const int32_t* table, int table_stride,
                                   const int32_t* positions, const int32_t* token_req,
                                   const int32_t* slots, int T, int nh, int nkv, int d, int dv,
                                   int page_size, int num_pages, float scale, int window,
                                   const float* slopes, int chunk, const float* sinks, int out_f32, int dtype,
                                   kvc_stream stream) {
  if (T < 0 || nh <= 0 || nkv <= 0 || page_size <= 0 || num_pages <= 0 || table_stride <= 0)
    return kvc_fail("kvc_paged_attention: bad sizes");
  if (nh % nkv) return kvc_fail("kvc_paged_attention: heads must be a multiple of kv heads");
  if (d <= 0 || d > kMaxHeadDim)
    return kvc_fail("kvc_paged_attention: head size must be positive, at most 512");
  if (dv <= 0 || dv > kMaxHeadDim)
    return kvc_fail("kvc_paged_attention: value size must be positive, at most 512");
  if (q_stride < static_cast<int64_t>(nh) * d)
    return kvc_fail("kvc_paged_attention: q stride too small");
  if (T == 0) return 0;
  const dim3 grid(T, (nh + kWavesPerBlock - 1) / kWavesPerBlock);
  if (d > kUsualHeadDim || dv > kUsualHeadDim) {
    KVC_DISPATCH_DTYPE(
        dtype, Tp,
        hipLaunchKernelGGL((paged_attention_wave_kernel<Tp, kMaxHeadDim>), grid, dim3(kWavesPerBlock * kWave), 0,
                           reinterpret_cast<hipStream_t>(stream), static_cast<Tp*>(out),
                           static_cast<const Tp*>(q), q_stride, static_cast<const Tp*>(k_cache),
                           static_cast<const Tp*>(v_cache), table, table_stride, positions,
                           token_req, slots, nh, nkv, d, dv, page_size, num_pages, scale, window, slopes,
                           chunk, sinks, out_f32));
    return kvc_check_launch("kvc_paged_attention");
  }
  KVC_DISPATCH_DTYPE(
      dtype, Tp,
      hipLaunchKernelGGL((paged_attention_wave_kernel<Tp, kUsualHeadDim>), grid, dim3(kWavesPerBlock * kWave), 0,
                         reinterpret_cast<hipStream_t>(stream), static_cast<Tp*>(out),
                         static_cast<const Tp*>(q), q_stride, static_cast<const Tp*>(k_cache),
                         static_cast<const Tp*>(v_cache), table, table_stride, positions,
                         token_req, slots, nh, nkv, d, dv, page_size, num_pages, scale, window, slopes,
                         chunk, sinks, out_f32));
  return kvc_check_launch("kvc_paged_attention");
}

// ------------------------------------- per-head norm, rotation and the K/V write in one
// One block of four waves per token; a wave takes one head at a time.  A q or k head of d
// elements is (optionally) divided by its root mean square, eps inside the root, and
// multiplied by a gain shared by all heads; then its first rot_dim elements are rotated
// (pairs (2j, 2j+1) when interleaved, (j, j + rot_dim/2) otherwise); all in float32, rounded
// once on the way out.  q heads go back in place, k heads in place and to K[page, kv head,
// offset, :]; the value heads of dv elements are copied to V[page, kv head, :, offset].
namespace {

constexpr int kMaxValuePlanes = 4;
template <typename T>
struct ValuePlanes {
  T* plane[kMaxValuePlanes];
};

template <typename T, int MAXD>
__global__ __launch_bounds__(256) void qk_norm_rope_kv_write_kernel(
    T* __restrict__ qkv, int64_t row_stride, T* __restrict__ k_cache, ValuePlanes<T> v_planes, int v_chunk,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_tab, const float* __restrict__ sin_tab, int rot_dim,
    int interleaved, const int32_t* __restrict__ kv_slot, int nh, int nkv, int d, int dv,
    int page_size, int write_kv, int copy_values) {
  __shared__ float head_s[4][MAXD];
  const int t = blockIdx.x;
  const int slot = kv_slot[t];
  if (slot == -2) return;  // padding token
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int half = rot_dim / 2;
  T* row = qkv + static_cast<int64_t>(t) * row_stride;
  const bool store_kv = write_kv && slot >= 0;
  const int page = store_kv ? slot / page_size : 0;
  const int off = store_kv ? slot - page * page_size : 0;
  const float* cs = cos_tab + static_cast<int64_t>(t) * half;
  const float* sn = sin_tab + static_cast<int64_t>(t) * half;

  // blockIdx.y deals the heads out four at a time (a wave each)
  for (int head_base = 4 * blockIdx.y; head_base < nh + nkv; head_base += 4 * gridDim.y) {
    const bool live = head_base + wave < nh + nkv;
    const int head = live ? head_base + wave : 0;
    T* hp = row + static_cast<int64_t>(head) * d;
    const float* gain = head < nh ? q_gain : k_gain;
    float x[MAXD / kWave];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAXD / kWave; ++i) {
      const int e = lane + i * kWave;
      x[i] = e < d ? to_float(hp[e]) : 0.f;
      ss = fmaf(x[i], x[i], ss);
    }
    if (gain != nullptr) {
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / static_cast<float>(d) + eps);
#pragma unroll
      for (int i = 0; i < MAXD / kWave; ++i) {
        const int e = lane + i * kWave;
        if (e < d) x[i] = x[i] * inv * gain[e];
      }
    }
#pragma unroll
    for (int i = 0; i < MAXD / kWave; ++i) {
      const int e = lane + i * kWave;
      if (e < d) head_s[wave][e] = x[i];
    }
    __syncthreads();
    T* kc = nullptr;
    if (live && head >= nh && store_kv)
      kc = k_cache + ((static_cast<int64_t>(page) * nkv + (head - nh)) * page_size + off) * d;
#pragma unroll
    for (int i = 0; i < MAXD / kWave; ++i) {
      const int e = lane + i * kWave;
      if (e >= d || !live) continue;
      float y = x[i];
      if (e < rot_dim) {
        int j, e0, e1;
        if (interleaved) {
          j = e >> 1; e0 = e & ~1; e1 = e0 + 1;
        } else {
          j = e < half ? e : e - half; e0 = j; e1 = j + half;
        }
        const float x0 = head_s[wave][e0], x1 = head_s[wave][e1];
        y = (e == e0) ? rotate_first(x0, x1, cs[j], sn[j]) : rotate_second(x0, x1, cs[j], sn[j]);
      }
      const T r = from_float<T>(y);
      hp[e] = r;
      if (kc != nullptr) kc[e] = r;
    }
    __syncthreads();
  }
  if (!store_kv || !copy_values) return;
  // element i of a value head goes to plane i / v_chunk, V[page, kv head, i % v_chunk, offset];
  // the token's blocks share the copy
  const T* vrow = row + static_cast<int64_t>(nh + nkv) * d;
  const int64_t v_base = static_cast<int64_t>(page) * nkv * page_size * v_chunk + off;
  for (int w = blockIdx.y * blockDim.x + threadIdx.x; w < nkv * dv; w += blockDim.x * gridDim.y) {
    const int head = w / dv, i = w - head * dv;
    const int c = i / v_chunk, ii = i - c * v_chunk;
    v_planes.plane[c][v_base + (static_cast<int64_t>(head) * v_chunk + ii) * page_size] = vrow[w];
  }
}

// The same norm, rotation and key write for heads of up to 64 elements: a wave per (token,
// head) with an element a lane; a rotary pair's partner is a lane away (its neighbour, or half
// the rotated width apart), so the wave needs neither LDS nor a barrier.  The values are left
// to the kernel below.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_k_write_small_kernel(
    T* __restrict__ qkv, int64_t row_stride, T* __restrict__ k_cache,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_tab, const float* __restrict__ sin_tab, int rot_dim,
    int interleaved, const int32_t* __restrict__ kv_slot, int num_tokens, int nh, int nkv, int d,
    int page_size, int write_kv) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  const int heads = nh + nkv;
  if (item >= static_cast<int64_t>(num_tokens) * heads) return;  // the whole wave
  const int t = static_cast<int>(item / heads);
  const int head = static_cast<int>(item - static_cast<int64_t>(t) * heads);
  const int slot = kv_slot[t];
  if (slot == -2) return;  // padding token
  const int half = rot_dim / 2;
  T* hp = qkv + static_cast<int64_t>(t) * row_stride + static_cast<int64_t>(head) * d;
  const bool in = lane < d;
  float x = in ? to_float(hp[lane]) : 0.f;
  const float* gain = head < nh ? q_gain : k_gain;
  if (gain != nullptr) {
    const float ss = wave_sum(x * x);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(d) + eps);
    if (in) x = x * inv * gain[lane];
  }
  // the pair's other element, from its lane (every lane takes part in the exchange)
  int partner, j;
  bool first;
  if (interleaved) {
    partner = lane ^ 1; j = lane >> 1; first = (lane & 1) == 0;
  } else {
    first = lane < half; j = first ? lane : lane - half; partner = first ? lane + half : lane - half;
  }
  const float other = __shfl(x, partner & (kWave - 1), kWave);
  float y = x;
  if (lane < rot_dim) {
    const float c = cos_tab[static_cast<int64_t>(t) * half + j], sn = sin_tab[static_cast<int64_t>(t) * half + j];
    y = first ? rotate_first(x, other, c, sn) : rotate_second(other, x, c, sn);
  }
  if (!in) return;
  const T r = from_float<T>(y);
  hp[lane] = r;
  if (head >= nh && write_kv && slot >= 0) {
    const int page = slot / page_size, off = slot - page * page_size;
    k_cache[((static_cast<int64_t>(page) * nkv + (head - nh)) * page_size + off) * d + lane] = r;
  }
}

// The values of eight consecutive tokens a block, for steps of many tokens.  A V page keeps the
// keys side by side, so a token alone stores its values two or four bytes at a time, page_size
// elements apart; when the block's eight tokens lie side by side in one page (a portion of a
// prompt mostly does), a thread gathers one element of all eight and stores them together.
template <typename T>
__global__ __launch_bounds__(256) void value_planes_write_tile_kernel(
    const T* __restrict__ qkv, int64_t row_stride, ValuePlanes<T> v_planes, int v_chunk,
    const int32_t* __restrict__ kv_slot, int num_tokens, int v_begin, int nkv, int dv, int page_size) {
  constexpr int TILE = 8;
  const int t0 = blockIdx.x * TILE;
  const int n_tok = (num_tokens - t0 < TILE) ? num_tokens - t0 : TILE;
  const int s0 = kv_slot[t0];
  bool side_by_side = n_tok == TILE && s0 >= 0 && (s0 & 7) == 0 && (page_size & 7) == 0;
  for (int ti = 1; ti < n_tok; ++ti) side_by_side = side_by_side && kv_slot[t0 + ti] == s0 + ti;
  if (side_by_side) {
    const int page = s0 / page_size, off = s0 - page * page_size;
    const int64_t v_base = static_cast<int64_t>(page) * nkv * page_size * v_chunk + off;
    for (int w = threadIdx.x; w < nkv * dv; w += blockDim.x) {
      const int head = w / dv, i = w - head * dv;
      const int c = i / v_chunk, ii = i - c * v_chunk;
      const T* src = qkv + static_cast<int64_t>(t0) * row_stride + v_begin + w;
      alignas(16) T vals[TILE];
#pragma unroll
      for (int ti = 0; ti < TILE; ++ti) vals[ti] = src[ti * row_stride];
      T* dst = v_planes.plane[c] + v_base + (static_cast<int64_t>(head) * v_chunk + ii) * page_size;
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(vals);
      if constexpr (sizeof(T) == 4) *reinterpret_cast<uint4*>(dst + 4) = *reinterpret_cast<const uint4*>(vals + 4);
    }
    return;
  }
  for (int w = threadIdx.x; w < n_tok * nkv * dv; w += blockDim.x) {
    const int ti = w / (nkv * dv), rest = w - ti * nkv * dv;
    const int slot = kv_slot[t0 + ti];
    if (slot < 0) continue;
    const int page = slot / page_size, off = slot - page * page_size;
    const int head = rest / dv, i = rest - head * dv;
    const int c = i / v_chunk, ii = i - c * v_chunk;
    v_planes.plane[c][static_cast<int64_t>(page) * nkv * page_size * v_chunk + off +
                      (static_cast<int64_t>(head) * v_chunk + ii) * page_size] =
        qkv[static_cast<int64_t>(t0 + ti) * row_stride + v_begin + rest];
  }
}

}  // namespace

extern "C" int kvc_qk_norm_rope_kv_write(void* qkv, int64_t row_stride, void* k_cache,
                                         void* const* host_v_planes, int num_v_planes,
                                         const float* q_gain, const float* k_gain, float eps,
                                         const float* cos_tab, const float* sin_tab, int rot_dim,
                                         int interleaved, const int32_t* kv_slot, int T, int nh,
                                         int nkv, int d, int dv, int page_size, int write_kv,
                                         int dtype, kvc_stream stream) {
  if (T < 0 || nh <= 0 || nkv <= 0 || d <= 0 || dv <= 0 || page_size <= 0)
    return kvc_fail("kvc_qk_norm_rope_kv_write: bad sizes");
  if (d > kMaxHeadDim) return kvc_fail("kvc_qk_norm_rope_kv_write: head size above 512");
  if (rot_dim < 0 || rot_dim > d || (rot_dim & 1))
    return kvc_fail("kvc_qk_norm_rope_kv_write: rot_dim must be even and at most the head size");
  if (row_stride < static_cast<int64_t>(nh + nkv) * d + static_cast<int64_t>(nkv) * dv)
    return kvc_fail("kvc_qk_norm_rope_kv_write: rows too short for the heads");
  if ((q_gain == nullptr) != (k_gain == nullptr))
    return kvc_fail("kvc_qk_norm_rope_kv_write: gains for both q and k, or for neither");
  if (num_v_planes < 1 || num_v_planes > kMaxValuePlanes || dv % num_v_planes)
    return kvc_fail("kvc_qk_norm_rope_kv_write: one to four value planes that divide the value size");
  if (T == 0) return 0;
  const int v_chunk = dv / num_v_planes;
  // a block per token and four heads (up to sixteen such blocks a token, which walk the heads
  // beyond): blocks enough also for a few tokens, and two barriers a block
  const int all_groups = (nh + nkv + 3) / 4;
  const int head_groups = all_groups < 16 ? all_groups : 16;
  // steps of many tokens store the values eight tokens at a time, 16 bytes a store (the planes
  // must be 16-byte aligned for that, which whole pages of 8 tokens and more are)
  bool tiled_values = write_kv && T >= 16 && page_size % 8 == 0;
  for (int c = 0; c < num_v_planes; ++c)
    tiled_values = tiled_values && (reinterpret_cast<uintptr_t>(host_v_planes[c]) & 15) == 0;
  if (tiled_values && d <= kWave) {
    // many tokens and heads of up to 64 elements: a wave a head, then the values
    const int64_t waves = static_cast<int64_t>(T) * (nh + nkv);
    KVC_DISPATCH_DTYPE(
        dtype, Tp, ValuePlanes<Tp> planes{};
        for (int c = 0; c < num_v_planes; ++c) planes.plane[c] = static_cast<Tp*>(host_v_planes[c]);
        hipLaunchKernelGGL(qk_norm_rope_k_write_small_kernel<Tp>, dim3(static_cast<unsigned>((waves + 3) / 4)),
                           dim3(256), 0, reinterpret_cast<hipStream_t>(stream), static_cast<Tp*>(qkv),
                           row_stride, static_cast<Tp*>(k_cache), q_gain, k_gain, eps, cos_tab, sin_tab,
                           rot_dim, interleaved, kv_slot, T, nh, nkv, d, page_size, write_kv);
        hipLaunchKernelGGL(value_planes_write_tile_kernel<Tp>, dim3((T + 7) / 8), dim3(256), 0,
                           reinterpret_cast<hipStream_t>(stream), static_cast<const Tp*>(qkv), row_stride,
                           planes, v_chunk, kv_slot, T, (nh + nkv) * d, nkv, dv, page_size));
    return kvc_check_launch("kvc_qk_norm_rope_kv_write");
  }
  if (d > kUsualHeadDim) {
    KVC_DISPATCH_DTYPE(
        dtype, Tp, ValuePlanes<Tp> planes{};
        for (int c = 0; c < num_v_planes; ++c) planes.plane[c] = static_cast<Tp*>(host_v_planes[c]);
        hipLaunchKernelGGL((qk_norm_rope_kv_write_kernel<Tp, kMaxHeadDim>), dim3(T, head_groups), dim3(256), 0,
                           reinterpret_cast<hipStream_t>(stream), static_cast<Tp*>(qkv), row_stride,
                           static_cast<Tp*>(k_cache), planes, v_chunk, q_gain, k_gain, eps,
                           cos_tab, sin_tab, rot_dim, interleaved, kv_slot, nh, nkv, d, dv, page_size,
                           write_kv, tiled_values ? 0 : 1);
        if (tiled_values) hipLaunchKernelGGL(
            value_planes_write_tile_kernel<Tp>, dim3((T + 7) / 8), dim3(256), 0,
            reinterpret_cast<hipStream_t>(stream), static_cast<const Tp*>(qkv), row_stride, planes,
            v_chunk, kv_slot, T, (nh + nkv) * d, nkv, dv, page_size));
    return kvc_check_launch("kvc_qk_norm_rope_kv_write");
  }
  KVC_DISPATCH_DTYPE(
      dtype, Tp, ValuePlanes<Tp> planes{};
      for (int c = 0; c < num_v_planes; ++c) planes.plane[c] = static_cast<Tp*>(host_v_planes[c]);
      hipLaunchKernelGGL((qk_norm_rope_kv_write_kernel<Tp, kUsualHeadDim>), dim3(T, head_groups), dim3(256), 0,
                         reinterpret_cast<hipStream_t>(stream), static_cast<Tp*>(qkv), row_stride,
                         static_cast<Tp*>(k_cache), planes, v_chunk, q_gain, k_gain, eps,
                         cos_tab, sin_tab, rot_dim, interleaved, kv_slot, nh, nkv, d, dv, page_size,
                         write_kv, tiled_values ? 0 : 1);
      if (tiled_values) hipLaunchKernelGGL(
          value_planes_write_tile_kernel<Tp>, dim3((T + 7) / 8), dim3(256), 0,
          reinterpret_cast<hipStream_t>(stream), static_cast<const Tp*>(qkv), row_stride, planes,
          v_chunk, kv_slot, T, (nh + nkv) * d, nkv, dv, page_size));
  return kvc_check_launch("kvc_qk_norm_rope_kv_write");
}
