// Mixers whose memory is a matrix per head, S [d, dv] in float32, carried from token to token
// (linear attention and its kin), and the small float32 kernels around them.
//
// kvc_linear_state_scan walks each request's tokens in order.  Two update rules:
//   key decay   S <- diag(a_t) S + k_t v_t^T                      (a_t one factor per key channel)
//   delta rule  S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T   (g_t, beta_t scalars)
//   scalar gates  S <- g_t S + beta_t k_t v_t^T                   (g_t, beta_t scalars per head)
// and in all o_t = S^T (q_scale q_t), read after the token's write.  A block owns one (request, head, tile
// of VT value channels); the NSL threads that share a column of the state are neighbouring lanes
// (their partial sums meet through lane permutations, in one fixed order) and each keeps NPT rows in
// registers; q, k, the factors and v of 16 tokens at a time go through LDS.  A request whose
// first token of the step is at position 0 starts from zero, any other from its slot's state;
// the state goes back to the slot at the end (kept there with its rows in fours: element (n, c) of a
// head at ((n / 4) * dv + c) * 4 + n % 4, the row count rounded up to a multiple of four).  What a token's result is depends on its request's
// earlier tokens only, not on how they were cut into steps or what else the batch holds.

#include <hip/hip_runtime.h>

#include <cstdlib>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

#define S(stream) reinterpret_cast<hipStream_t>(stream)

constexpr int LSC = 16;  // tokens a stage

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_ff(float x) { return x / (1.f + expf(-x)); }
// log(1 + e^x) without a threshold: max(x, 0) + log1p(e^-|x|)
__device__ __forceinline__ float softplus_ff(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
// log(sigmoid(x)) = -softplus(-x)
__device__ __forceinline__ float log_sigmoid_f(float x) { return -softplus_ff(-x); }

// The sum of a value over the NSL (4 or 16) neighbouring lanes that share a column, by lane
// permutations inside a row of 16 lanes (no trip through LDS): neighbours in a quad, the quads of a
// half row, the two halves.  Every lane of the group ends with the same bits.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int NSL>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(NSL == 4 || NSL == 16, "columns are shared by 4 or by 16 lanes");
  v += dpp_f<0xB1>(v);  // quad_perm [1, 0, 3, 2]
  v += dpp_f<0x4E>(v);  // quad_perm [2, 3, 0, 1]
  if (NSL == 16) {
    v += dpp_f<0x141>(v);  // row_half_mirror
    v += dpp_f<0x140>(v);  // row_mirror
  }
  return v;
}

template <int NPT, int DELTA, int NSL, int FULL, int PF>
__global__ __launch_bounds__(256) void linear_state_scan_kernel(
    float* __restrict__ out, const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k,
    int64_t k_stride, const float* __restrict__ v, int64_t v_stride, const float* __restrict__ decay,
    int64_t decay_stride, const float* __restrict__ beta, int64_t beta_stride, float* __restrict__ state,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int nh, int nqk, int d,
    int dv, float q_scale, int scalar_gates, int ones_column) {
  constexpr int VT = 256 / NSL;  // value channels a block
  // with ones_column the rows of v hold dv - 1 values a head and the last column of the state's dv
  // takes a one for every token (a normaliser kept beside the matrix)
  const int dvin = dv - ones_column;
  // FULL: d == NPT * NSL, so no row needs a bound, and a thread's rows of q, k and the factors lie
  // side by side in LDS (row n of a token at (n % NSL) * NPT + n / NSL), read 16 bytes at a time
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int r = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * VT;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int ns = tid % NSL, pl = tid / NSL;
  const int c = c0 + pl;
  const bool c_ok = c < dv;
  const int width = nh * dv;
  const int b = q_start[r], e = q_start[r + 1];
  if (e <= b) return;
  if (token_req[b] < 0) {  // padding rows: zeros out, no state touched
    for (int idx = tid; idx < (e - b) * VT; idx += nthreads) {
      const int tt = idx / VT, cc = c0 + idx - tt * VT;
      if (cc < dv) out[static_cast<int64_t>(b + tt) * width + h * dv + cc] = 0.f;
    }
    return;
  }
  const int hk = h / (nh / nqk);
  // a head's state in memory: rows in fours, [ceil(d / 4)][dv][4], so that the four lanes that share a
  // column (and their neighbours' columns) read and write one contiguous run
  const int dpad = (d + 3) & ~3;
  float* st = state + (static_cast<int64_t>(slots[r]) * nh + h) * dpad * dv;
  auto st_at = [&](int n) -> int64_t { return (static_cast<int64_t>(n >> 2) * dv + c) * 4 + (n & 3); };
  const bool fresh = positions[b] == 0;
  float s[NPT];
  if (!fresh) {  // the same for the whole block
    // every row is asked for with no branch between the loads (a row or column that is not there
    // reads one that is, and is then set to zero), so that all of them are in flight together
    const int c_safe = c_ok ? c : dv - 1;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const int n = ns + NSL * i;
      const int n_safe = (FULL || n < d) ? n : 0;
      s[i] = st[(static_cast<int64_t>(n_safe >> 2) * dv + c_safe) * 4 + (n_safe & 3)];
    }
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      if (!c_ok || !(FULL || ns + NSL * i < d)) s[i] = 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < NPT; ++i) s[i] = 0.f;
  }
  // one stage's tokens, from the LDS buffers given
  auto work_stage = [&](const float* q_s, const float* k_s, const float* a_s, const float* v_s, int t0, int nt) {
    auto token = [&](int tt) {
      const float* qt = q_s + tt * d + (FULL ? ns * NPT : ns);
      const float* kt = k_s + tt * d + (FULL ? ns * NPT : ns);
      constexpr int ST = FULL ? 1 : NSL;  // from one of the thread's rows to its next, in LDS
      const float vv = v_s[tt * VT + pl];
      float acc = 0.f;
      if (DELTA && scalar_gates) {  // the same for the whole grid: S <- g S + (beta k) v^T
        const float g = a_s[2 * tt], bv = a_s[2 * tt + 1] * vv;
        float acc1 = 0.f;
#pragma unroll
        for (int i = 0; i < NPT; i += 2) {
          const int n = ns + NSL * i;
          if (FULL || n < d) {
            s[i] = fmaf(g, s[i], kt[ST * i] * bv);
            acc = fmaf(s[i], qt[ST * i], acc);
          }
          if (FULL || n + NSL < d) {
            s[i + 1] = fmaf(g, s[i + 1], kt[ST * (i + 1)] * bv);
            acc1 = fmaf(s[i + 1], qt[ST * (i + 1)], acc1);
          }
        }
        acc += acc1;
      } else if (DELTA) {
        const float g = a_s[2 * tt], bt = a_s[2 * tt + 1];
        float kd0 = 0.f, kd1 = 0.f;  // two running sums: half as long a chain of dependent operations
#pragma unroll
        for (int i = 0; i < NPT; i += 2) {
          const int n = ns + NSL * i;
          if (FULL || n < d) {
            s[i] *= g;
            kd0 = fmaf(s[i], kt[ST * i], kd0);
          }
          if (FULL || n + NSL < d) {
            s[i + 1] *= g;
            kd1 = fmaf(s[i + 1], kt[ST * (i + 1)], kd1);
          }
        }
        const float kd = group_sum<NSL>(kd0 + kd1);
        const float u = bt * (vv - kd);
        float acc1 = 0.f;
#pragma unroll
        for (int i = 0; i < NPT; i += 2) {
          const int n = ns + NSL * i;
          if (FULL || n < d) {
            s[i] = fmaf(kt[ST * i], u, s[i]);
            acc = fmaf(s[i], qt[ST * i], acc);
          }
          if (FULL || n + NSL < d) {
            s[i + 1] = fmaf(kt[ST * (i + 1)], u, s[i + 1]);
            acc1 = fmaf(s[i + 1], qt[ST * (i + 1)], acc1);
          }
        }
        acc += acc1;
      } else {
        const float* at = a_s + tt * d + (FULL ? ns * NPT : ns);
        float acc1 = 0.f;
#pragma unroll
        for (int i = 0; i < NPT; i += 2) {
          const int n = ns + NSL * i;
          if (FULL || n < d) {
            s[i] = fmaf(at[ST * i], s[i], kt[ST * i] * vv);
            acc = fmaf(s[i], qt[ST * i], acc);
          }
          if (FULL || n + NSL < d) {
            s[i + 1] = fmaf(at[ST * (i + 1)], s[i + 1], kt[ST * (i + 1)] * vv);
            acc1 = fmaf(s[i + 1], qt[ST * (i + 1)], acc1);
          }
        }
        acc += acc1;
      }
      acc = group_sum<NSL>(acc);
      if (ns == 0 && c_ok) out[static_cast<int64_t>(t0 + tt) * width + h * dv + c] = acc;
    };
    if (nt == LSC) {
      // a whole stage: unrolled, so that a token's LDS reads are under way while the token before
      // it is still being worked on (only the state itself passes from token to token)
#pragma unroll 4
      for (int tt = 0; tt < LSC; ++tt) token(tt);
    } else {
      for (int tt = 0; tt < nt; ++tt) token(tt);
    }
  };
  if constexpr (PF) {
    // Two sets of LDS buffers: while a stage is worked on, the next stage's q, k, factors and v are on
    // their way from memory into registers, and go into the other set afterwards (a block has one
    // wave a SIMD and nothing else to hide that latency behind).
    constexpr int QN = LSC * NPT * NSL / 256;  // values of q (and of k) a thread brings a stage
    constexpr int VN = LSC * VT / 256;
    const int set = 2 * LSC * d + LSC * (DELTA ? 2 : d) + LSC * VT;
    float qn[QN], kn[QN], an[DELTA ? 2 : QN], vn[VN];
    auto fetch = [&](int t0, int nt) {
#pragma unroll
      for (int j = 0; j < QN; ++j) {
        const int idx = tid + 256 * j, tt = idx / d, n = idx - tt * d;
        const int64_t t = t0 + (tt < nt ? tt : 0);
        qn[j] = q[t * q_stride + hk * d + n] * q_scale;
        kn[j] = k[t * k_stride + hk * d + n];
        if (!DELTA) an[j] = decay[t * decay_stride + h * d + n];
      }
      if (DELTA) {
        const int64_t t = t0 + (tid < nt ? tid : 0);
        an[0] = decay[t * decay_stride + h];
        an[1] = beta[t * beta_stride + h];
      }
#pragma unroll
      for (int j = 0; j < VN; ++j) {
        const int idx = tid + 256 * j, tt = idx / VT, cc = c0 + idx - tt * VT;
        const int64_t t = t0 + (tt < nt ? tt : 0);
        vn[j] = cc < dvin ? v[t * v_stride + h * dvin + cc] : (cc < dv ? 1.f : 0.f);
      }
    };
    auto stash = [&](float* base) {
      float* q_s = base;
      float* k_s = q_s + LSC * d;
      float* a_s = k_s + LSC * d;
      float* v_s = a_s + LSC * (DELTA ? 2 : d);
#pragma unroll
      for (int j = 0; j < QN; ++j) {
        const int idx = tid + 256 * j, tt = idx / d, n = idx - tt * d;
        const int at = tt * d + (n % NSL) * NPT + n / NSL;
        q_s[at] = qn[j];
        k_s[at] = kn[j];
        if (!DELTA) a_s[at] = an[j];
      }
      if (DELTA && tid < LSC) {
        a_s[2 * tid] = an[0];
        a_s[2 * tid + 1] = an[1];
      }
#pragma unroll
      for (int j = 0; j < VN; ++j) v_s[tid + 256 * j] = vn[j];
    };
    fetch(b, (e - b < LSC) ? e - b : LSC);
    stash(lds);
    __syncthreads();
    int which = 0;
    for (int t0 = b; t0 < e; t0 += LSC) {
      const int nt = (e - t0 < LSC) ? e - t0 : LSC;
      const bool more = t0 + LSC < e;
      if (more) fetch(t0 + LSC, (e - t0 - LSC < LSC) ? e - t0 - LSC : LSC);
      float* base = lds + which * set;
      work_stage(base, base + LSC * d, base + 2 * LSC * d, base + 2 * LSC * d + LSC * (DELTA ? 2 : d), t0, nt);
      if (more) stash(lds + (which ^ 1) * set);
      __syncthreads();
      which ^= 1;
    }
  } else {
    float* q_s = lds;               // [LSC][d]
    float* k_s = q_s + LSC * d;     // [LSC][d]
    float* a_s = k_s + LSC * d;     // [LSC][d] (key decay) or [LSC][2] (delta: g, beta)
    float* v_s = a_s + LSC * (DELTA ? 2 : d);  // [LSC][VT]
    for (int t0 = b; t0 < e; t0 += LSC) {
      const int nt = (e - t0 < LSC) ? e - t0 : LSC;
      __syncthreads();
      for (int idx = tid; idx < nt * d; idx += nthreads) {
        const int tt = idx / d, n = idx - tt * d;
        const int64_t t = t0 + tt;
        const int at = FULL ? tt * d + (n % NSL) * NPT + n / NSL : idx;
        q_s[at] = q[t * q_stride + hk * d + n] * q_scale;
        k_s[at] = k[t * k_stride + hk * d + n];
        if (!DELTA) a_s[at] = decay[t * decay_stride + h * d + n];
      }
      if (DELTA) {
        for (int tt = tid; tt < nt; tt += nthreads) {
          a_s[2 * tt] = decay[static_cast<int64_t>(t0 + tt) * decay_stride + h];
          a_s[2 * tt + 1] = beta[static_cast<int64_t>(t0 + tt) * beta_stride + h];
        }
      }
      for (int idx = tid; idx < nt * VT; idx += nthreads) {
        const int tt = idx / VT, cc = c0 + idx - tt * VT;
        v_s[idx] = cc < dvin ? v[static_cast<int64_t>(t0 + tt) * v_stride + h * dvin + cc] : (cc < dv ? 1.f : 0.f);
      }
      __syncthreads();
      work_stage(q_s, k_s, a_s, v_s, t0, nt);
    }
  }
  if (!c_ok) return;
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int n = ns + NSL * i;
    if (n < d) st[st_at(n)] = s[i];
  }
}

// a[t, i] = exp(log(sigmoid(z[t, i] + bias[i])) * inv_tau): sigmoid(z)^(1/tau), through its logarithm
__global__ __launch_bounds__(256) void sigmoid_power_kernel(float* __restrict__ a, const float* __restrict__ z,
                                                             int64_t z_stride, const float* __restrict__ bias,
                                                             float inv_tau, int T, int W) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<int64_t>(T) * W) return;
  const int t = static_cast<int>(idx / W), i = static_cast<int>(idx - static_cast<int64_t>(t) * W);
  const float x = z[t * z_stride + i] + (bias != nullptr ? bias[i] : 0.f);
  a[idx] = expf(log_sigmoid_f(x) * inv_tau);
}

// g[t, h] = exp(-exp(a_log[h]) * softplus(a_raw[t, h] + dt_bias[h])); beta[t, h] = sigmoid(b_raw[t, h])
__global__ __launch_bounds__(256) void decay_and_write_gates_kernel(
    float* __restrict__ g, float* __restrict__ beta, const float* __restrict__ a_raw, int64_t a_stride,
    const float* __restrict__ b_raw, int64_t b_stride, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, int T, int nh) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * nh) return;
  const int t = idx / nh, h = idx - t * nh;
  g[idx] = expf(-expf(a_log[h]) * softplus_ff(a_raw[t * a_stride + h] + dt_bias[h]));
  beta[idx] = sigmoid_f(b_raw[t * b_stride + h]);
}

// Heads of d float32 values made unit vectors in place, x / sqrt(sum x^2 + eps) * scale (the first
// first_heads heads times first_scale instead): a wave a (token, head).
__global__ __launch_bounds__(256) void unit_heads_kernel(float* __restrict__ x, int64_t stride, int T, int heads,
                                                         int d, float eps, float scale, int first_heads,
                                                         float first_scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (item >= static_cast<int64_t>(T) * heads) return;
  const int t = static_cast<int>(item / heads), h = static_cast<int>(item - static_cast<int64_t>(t) * heads);
  float* p = x + t * stride + static_cast<int64_t>(h) * d;
  float ss = 0.f;
  for (int i = lane; i < d; i += kWave) ss = fmaf(p[i], p[i], ss);
  ss = wave_sum(ss);
  const float inv = (h < first_heads ? first_scale : scale) / sqrtf(ss + eps);
  for (int i = lane; i < d; i += kWave) p[i] *= inv;
}

// out[t, h, c] = o[t, h, c] / sqrt(mean_c o^2 + eps) * gain[c] * silu(gate[t, h, c]): the norm of
// every head first, then the gate.  A wave a (token, head).
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void head_rmsnorm_gate_kernel(
    TO* __restrict__ out, const float* __restrict__ o, const TG* __restrict__ gate, int64_t gate_stride,
    const float* __restrict__ gain, float eps, int T, int heads, int dv) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (item >= static_cast<int64_t>(T) * heads) return;
  const int t = static_cast<int>(item / heads), h = static_cast<int>(item - static_cast<int64_t>(t) * heads);
  const float* p = o + (static_cast<int64_t>(t) * heads + h) * dv;
  const TG* gp = gate + t * gate_stride + static_cast<int64_t>(h) * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += kWave) ss = fmaf(p[i], p[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(dv) + eps);
  TO* op = out + (static_cast<int64_t>(t) * heads + h) * dv;
  for (int i = lane; i < dv; i += kWave)
    op[i] = from_float<TO>(p[i] * inv * gain[i] * silu_ff(to_float(gp[i])));
}


// The log gates of a matrix memory with a running maximum (mLSTM), for every request's tokens in
// order: i = cap tanh((i_raw + bi) / cap), f = logsigmoid(cap tanh((f_raw + bf) / cap)),
// m_t = max(f_t + m_(t-1), i_t), keep_t = exp(f_t + m_(t-1) - m_t), take_t = exp(i_t - m_t).
// A wave a (request, head).  The step m -> max(m + f, i) composes: a run of tokens acts as
// m -> max(m + A, B) with A the sum of its f and B the maximum it reaches from minus infinity.  So
// each lane takes a run of consecutive tokens, finds its (A, B), the runs are joined lane by lane
// from the request's m, and each lane walks its run again from where it starts: a chain of two
// runs and 64 joins instead of one of all tokens.  m starts at 0 at position 0 and otherwise comes
// from the slot's state, where the last one goes back.
template <int GATES_MADE>
__global__ __launch_bounds__(256) void max_gates_kernel(
    float* __restrict__ keep, float* __restrict__ take, float* __restrict__ m_out, const float* __restrict__ i_raw,
    int64_t i_stride, const float* __restrict__ f_raw, int64_t f_stride, const float* __restrict__ i_bias,
    const float* __restrict__ f_bias, float cap, float* __restrict__ m_state, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ token_req, const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots,
    int nh) {
  const int r = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int h_raw = blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int h = h_raw < nh ? h_raw : nh - 1;  // a wave beyond the heads only keeps the barrier's count
  const int b = q_start[r], e = q_start[r + 1];
  if (e <= b) return;
  const int n = e - b;
  const int run = (n + kWave - 1) / kWave;
  const int lo = b + (lane * run < n ? lane * run : n);
  const int hi = b + ((lane + 1) * run < n ? (lane + 1) * run : n);
  if (token_req[b] < 0) {  // padding rows
    for (int64_t t = lo; t < hi && h_raw < nh; ++t) {
      keep[t * nh + h] = 0.f;
      take[t * nh + h] = 0.f;
      m_out[t * nh + h] = 0.f;
    }
    return;
  }
  if (h_raw >= nh) {  // the whole wave
    __syncthreads();
    return;
  }
  const float inv_cap = 1.f / cap, bi = i_bias[h], bf = f_bias[h];
  // the log gates of all tokens first, dealt to the lanes one by one (nothing passes from token
  // to token here, so the loads of several are in flight together); they stay in keep and take
  // until the maxima are known
  if (!GATES_MADE) {
#pragma unroll 4
    for (int64_t t = b + lane; t < e; t += kWave) {
      take[t * nh + h] = cap * tanhf((i_raw[t * i_stride + h] + bi) * inv_cap);
      keep[t * nh + h] = log_sigmoid_f(cap * tanhf((f_raw[t * f_stride + h] + bf) * inv_cap));
    }
  }
  __syncthreads();  // the block's waves have one request: all of them arrive
  float A = 0.f, B = -INFINITY;  // an empty run leaves m as it is
#pragma unroll 4
  for (int64_t t = lo; t < hi; ++t) {
    const float gf = keep[t * nh + h], gi = take[t * nh + h];
    A += gf;
    B = fmaxf(B + gf, gi);
  }
  float* ms = m_state + static_cast<int64_t>(slots[r]) * nh + h;
  float m = positions[b] == 0 ? 0.f : *ms;
  float mine = m;
  const int runs = (n + run - 1) / run;  // lanes whose run holds a token: one for a single token
  for (int l = 0; l < runs; ++l) {
    if (l == lane) mine = m;
    m = fmaxf(m + __shfl(A, l, kWave), __shfl(B, l, kWave));
  }
  if (lane == 0) *ms = m;
  for (int64_t t = lo; t < hi; ++t) {
    const float gf = keep[t * nh + h], gi = take[t * nh + h];
    const float next = fmaxf(gf + mine, gi);
    keep[t * nh + h] = expf(gf + mine - next);
    take[t * nh + h] = expf(gi - next);
    m_out[t * nh + h] = next;
    mine = next;
  }
}

// The log gates alone, a thread a (token, head): what max_gates_kernel<1> starts from.  With many
// tokens a request the tanh, logarithm and exponential of every gate are most of the work, and
// a wave a (request, head) would leave the chip idle.
__global__ __launch_bounds__(256) void log_gates_kernel(float* __restrict__ keep, float* __restrict__ take,
                                                         const float* __restrict__ i_raw, int64_t i_stride,
                                                         const float* __restrict__ f_raw, int64_t f_stride,
                                                         const float* __restrict__ i_bias,
                                                         const float* __restrict__ f_bias, float cap, int64_t total,
                                                         int nh) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int64_t t = idx / nh;
  const int h = static_cast<int>(idx - t * nh);
  const float inv_cap = 1.f / cap;
  take[idx] = cap * tanhf((i_raw[t * i_stride + h] + i_bias[h]) * inv_cap);
  keep[idx] = log_sigmoid_f(cap * tanhf((f_raw[t * f_stride + h] + f_bias[h]) * inv_cap));
}

// The end of the same mixer: o[t, h, :dv] and the normaliser's product with the query at column dv
// of each head's dv + 1 columns.  y = o / (max(|n.q|, exp(-m)) + den_eps); y over its root mean
// square (eps inside the root) times gain[h * dv + c] times sigmoid(gate[t, h, c]).  A wave a
// (token, head).
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void max_gated_finish_kernel(
    TO* __restrict__ out, const float* __restrict__ o, const float* __restrict__ m, const TG* __restrict__ gate,
    int64_t gate_stride, const float* __restrict__ gain, float eps, float den_eps, int T, int heads, int dv) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (item >= static_cast<int64_t>(T) * heads) return;
  const int t = static_cast<int>(item / heads), h = static_cast<int>(item - static_cast<int64_t>(t) * heads);
  const float* p = o + item * (dv + 1);
  const TG* gp = gate + t * gate_stride + static_cast<int64_t>(h) * dv;
  const float den = fmaxf(fabsf(p[dv]), expf(-m[item])) + den_eps;
  float ss = 0.f;
  for (int i = lane; i < dv; i += kWave) {
    const float y = p[i] / den;
    ss = fmaf(y, y, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(dv) + eps);
  TO* op = out + item * dv;
  const float* gn = gain + static_cast<int64_t>(h) * dv;
  for (int i = lane; i < dv; i += kWave)
    op[i] = from_float<TO>(p[i] / den * inv * gn[i] * sigmoid_f(to_float(gp[i])));
}

}  // namespace

extern "C" int kvc_max_gates(float* keep, float* take, float* m_out, const float* i_raw, int64_t i_stride,
                             const float* f_raw, int64_t f_stride, const float* i_bias, const float* f_bias,
                             float cap, float* m_state, const int32_t* positions, const int32_t* token_req,
                             const int32_t* q_start, const int32_t* slots, int T, int R, int nh,
                             kvc_stream stream) {
  if (T < 0 || R < 0 || nh <= 0 || i_stride < nh || f_stride < nh || !(cap > 0.f))
    return kvc_fail("kvc_max_gates: bad sizes");
  if (R == 0 || T == 0) return 0;
  if (T > 2 * R) {  // portions of prompts: the gates by all threads first, then the walk of the maxima
    const int64_t total = static_cast<int64_t>(T) * nh;
    hipLaunchKernelGGL(log_gates_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, S(stream),
                       keep, take, i_raw, i_stride, f_raw, f_stride, i_bias, f_bias, cap, total, nh);
    hipLaunchKernelGGL(max_gates_kernel<1>, dim3(R, (nh + 3) / 4), dim3(256), 0, S(stream), keep, take, m_out, i_raw,
                       i_stride, f_raw, f_stride, i_bias, f_bias, cap, m_state, positions, token_req, q_start, slots,
                       nh);
    return kvc_check_launch("kvc_max_gates");
  }
  // four waves a block, a wave a (request, head)
  hipLaunchKernelGGL(max_gates_kernel<0>, dim3(R, (nh + 3) / 4), dim3(256), 0, S(stream), keep, take, m_out, i_raw, i_stride, f_raw,
                     f_stride, i_bias, f_bias, cap, m_state, positions, token_req, q_start, slots, nh);
  return kvc_check_launch("kvc_max_gates");
}

extern "C" int kvc_max_gated_finish(void* out, int out_dtype, const float* o, const float* m, const void* gate,
                                    int64_t gate_stride, int gate_dtype, const float* gain, float eps,
                                    float den_eps, int T, int heads, int dv, kvc_stream stream) {
  if (T < 0 || heads <= 0 || dv <= 0 || gate_stride < static_cast<int64_t>(heads) * dv)
    return kvc_fail("kvc_max_gated_finish: bad sizes");
  if (T == 0) return 0;
  const int64_t waves = static_cast<int64_t>(T) * heads;
  const dim3 grid(static_cast<unsigned>((waves + 3) / 4));
#define KVC_MGF(TG, TO)                                                                                        \
  hipLaunchKernelGGL((max_gated_finish_kernel<TG, TO>), grid, dim3(256), 0, S(stream), static_cast<TO*>(out), o, m, \
                     static_cast<const TG*>(gate), gate_stride, gain, eps, den_eps, T, heads, dv)
  if (gate_dtype == 0 && out_dtype == 0) {
    KVC_MGF(float, float);
  } else if (gate_dtype == 0 && out_dtype == 1) {
    KVC_MGF(float, bf16_t);
  } else if (gate_dtype == 1 && out_dtype == 1) {
    KVC_MGF(bf16_t, bf16_t);
  } else if (gate_dtype == 1 && out_dtype == 0) {
    KVC_MGF(bf16_t, float);
  } else {
    return kvc_fail("kvc_max_gated_finish: unknown dtype code");
  }
#undef KVC_MGF
  return kvc_check_launch("kvc_max_gated_finish");
}

extern "C" int kvc_linear_state_scan(float* out, const float* q, int64_t q_stride, const float* k,
                                     int64_t k_stride, const float* v, int64_t v_stride,
                                     const float* decay, int64_t decay_stride, const float* beta,
                                     int64_t beta_stride, float* state, const int32_t* positions,
                                     const int32_t* token_req, const int32_t* q_start,
                                     const int32_t* slots, int R, int nh, int nqk, int d, int dv,
                                     int rule, float q_scale, int ones_column,
                                     kvc_stream stream) {
  ones_column = ones_column ? 1 : 0;
  if (rule < 0 || rule > 2) return kvc_fail("kvc_linear_state_scan: the rule is 0 (key decay), 1 (delta) or 2 (scalar gates)");
  const int delta_rule = rule != 0;  // a gate and a factor per head and token instead of a decay per key channel
  const int scalar_gates = rule == 2;
  if (R < 0 || nh <= 0 || nqk <= 0 || nh % nqk || d <= 0 || dv <= 0)
    return kvc_fail("kvc_linear_state_scan: bad sizes");
  if (d > 256) return kvc_fail("kvc_linear_state_scan: at most 256 key channels a head");
  if (delta_rule && beta == nullptr) return kvc_fail("kvc_linear_state_scan: this rule needs beta");
  if (delta_rule && beta_stride < nh) return kvc_fail("kvc_linear_state_scan: rows of beta too short for the heads");
  if (q_stride < static_cast<int64_t>(nqk) * d || k_stride < static_cast<int64_t>(nqk) * d ||
      v_stride < static_cast<int64_t>(nh) * (dv - ones_column) || dv - ones_column <= 0 || decay_stride < (delta_rule ? nh : static_cast<int64_t>(nh) * d))
    return kvc_fail("kvc_linear_state_scan: rows too short for the heads");
  if (R == 0) return 0;
  // tiles of 64 value channels with 4 threads a column, or, where that leaves compute units
  // without a block, tiles of 16 with 16 threads a column
  const int64_t wide_blocks = static_cast<int64_t>(R) * nh * ((dv + 63) / 64);
  const bool narrow = dv < 64 || wide_blocks < kvc_device_compute_units();
  const int NSL = narrow ? 16 : 4, VT = 256 / NSL;
  const dim3 grid(R, nh, (dv + VT - 1) / VT);
  if (grid.y > 65535u || grid.z > 65535u) return kvc_fail("kvc_linear_state_scan: grid too large");
  const size_t lds = sizeof(float) * (2 * LSC * d + LSC * (delta_rule ? 2 : d) + LSC * VT);
  const int per_thread = (d + NSL - 1) / NSL;
  static const bool no_pf = getenv("KVC_LSCAN_NOPF") != nullptr;  // for tuning
#define KVC_LSCAN_F(NPT, DELTA, NSL_, FULL_, PF_)                                                             \
  hipLaunchKernelGGL((linear_state_scan_kernel<NPT, DELTA, NSL_, FULL_, PF_>), grid, dim3(256),               \
                     lds*(PF_ ? 2 : 1), S(stream), out, q, q_stride, k, k_stride, v, v_stride, decay,         \
                     decay_stride, beta, beta_stride, state, positions, token_req, q_start, slots, nh, nqk, d, \
                     dv, q_scale, scalar_gates, ones_column)
  // two sets of LDS buffers (the next stage fetched while one is worked on) where a stage's values
  // deal out evenly to the threads and both sets fit the 64 KB a block may take
#define KVC_LSCAN(NPT, DELTA, NSL_)                                                  \
  do {                                                                               \
    if (d == NPT * NSL_ && (NPT * NSL_) % 16 == 0 && 2 * lds <= 64 * 1024 && !no_pf) {  \
      KVC_LSCAN_F(NPT, DELTA, NSL_, 1, ((NPT * NSL_) % 16 == 0 ? 1 : 0));            \
    } else if (d == NPT * NSL_) {                                                    \
      KVC_LSCAN_F(NPT, DELTA, NSL_, 1, 0);                                           \
    } else {                                                                         \
      KVC_LSCAN_F(NPT, DELTA, NSL_, 0, 0);                                           \
    }                                                                                \
  } while (0)
#define KVC_LSCAN_N(NPT)                 \
  do {                                   \
    if (delta_rule && narrow) {          \
      KVC_LSCAN(NPT, 1, 16);             \
    } else if (delta_rule) {             \
      KVC_LSCAN(NPT, 1, 4);              \
    } else if (narrow) {                 \
      KVC_LSCAN(NPT, 0, 16);             \
    } else {                             \
      KVC_LSCAN(NPT, 0, 4);              \
    }                                    \
  } while (0)
  if (per_thread <= 2) {
    KVC_LSCAN_N(2);
  } else if (per_thread <= 4) {
    KVC_LSCAN_N(4);
  } else if (per_thread <= 8) {
    KVC_LSCAN_N(8);
  } else if (per_thread <= 16) {
    KVC_LSCAN_N(16);
  } else if (per_thread <= 32) {
    KVC_LSCAN_N(32);
  } else {
    KVC_LSCAN_N(64);
  }
#undef KVC_LSCAN_N
#undef KVC_LSCAN
#undef KVC_LSCAN_F
  return kvc_check_launch("kvc_linear_state_scan");
}

extern "C" int kvc_sigmoid_power(float* a, const float* z, int64_t z_stride, const float* bias,
                                 float inv_tau, int T, int W, kvc_stream stream) {
  if (T < 0 || W <= 0 || z_stride < W) return kvc_fail("kvc_sigmoid_power: bad sizes");
  if (T == 0) return 0;
  const int64_t n = static_cast<int64_t>(T) * W;
  hipLaunchKernelGGL(sigmoid_power_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, S(stream),
                     a, z, z_stride, bias, inv_tau, T, W);
  return kvc_check_launch("kvc_sigmoid_power");
}

extern "C" int kvc_decay_and_write_gates(float* g, float* beta, const float* a_raw, int64_t a_stride,
                                         const float* b_raw, int64_t b_stride, const float* a_log,
                                         const float* dt_bias, int T, int nh, kvc_stream stream) {
  if (T < 0 || nh <= 0 || a_stride < nh || b_stride < nh) return kvc_fail("kvc_decay_and_write_gates: bad sizes");
  if (T == 0) return 0;
  hipLaunchKernelGGL(decay_and_write_gates_kernel, dim3((T * nh + 255) / 256), dim3(256), 0, S(stream), g, beta,
                     a_raw, a_stride, b_raw, b_stride, a_log, dt_bias, T, nh);
  return kvc_check_launch("kvc_decay_and_write_gates");
}

extern "C" int kvc_unit_heads(float* x, int64_t stride, int T, int heads, int d, float eps, float scale,
                              int first_heads, float first_scale, kvc_stream stream) {
  if (T < 0 || heads <= 0 || d <= 0 || stride < static_cast<int64_t>(heads) * d)
    return kvc_fail("kvc_unit_heads: bad sizes");
  if (T == 0) return 0;
  const int64_t waves = static_cast<int64_t>(T) * heads;
  hipLaunchKernelGGL(unit_heads_kernel, dim3(static_cast<unsigned>((waves + 3) / 4)), dim3(256), 0, S(stream), x,
                     stride, T, heads, d, eps, scale, first_heads, first_scale);
  return kvc_check_launch("kvc_unit_heads");
}

extern "C" int kvc_head_rmsnorm_gate(void* out, int out_dtype, const float* o, const void* gate,
                                     int64_t gate_stride, int gate_dtype, const float* gain, float eps,
                                     int T, int heads, int dv, kvc_stream stream) {
  if (T < 0 || heads <= 0 || dv <= 0 || gate_stride < static_cast<int64_t>(heads) * dv)
    return kvc_fail("kvc_head_rmsnorm_gate: bad sizes");
  if (T == 0) return 0;
  const int64_t waves = static_cast<int64_t>(T) * heads;
  const dim3 grid(static_cast<unsigned>((waves + 3) / 4));
#define KVC_HRG(TG, TO)                                                                                  \
  hipLaunchKernelGGL((head_rmsnorm_gate_kernel<TG, TO>), grid, dim3(256), 0, S(stream), static_cast<TO*>(out), o, \
                     static_cast<const TG*>(gate), gate_stride, gain, eps, T, heads, dv)
  if (gate_dtype == 0 && out_dtype == 0) {
    KVC_HRG(float, float);
  } else if (gate_dtype == 0 && out_dtype == 1) {
    KVC_HRG(float, bf16_t);
  } else if (gate_dtype == 1 && out_dtype == 1) {
    KVC_HRG(bf16_t, bf16_t);
  } else if (gate_dtype == 1 && out_dtype == 0) {
    KVC_HRG(bf16_t, float);
  } else {
    return kvc_fail("kvc_head_rmsnorm_gate: unknown dtype code");
  }
#undef KVC_HRG
  return kvc_check_launch("kvc_head_rmsnorm_gate");
}
