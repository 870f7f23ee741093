// Routed experts: the router's choice, the arrangement of (token, choice) pairs by expert, the
// experts' two products over their own rows, and the weighted sum.
//
// Everything is decided on the device and every grid is sized by bounds known on the host (pairs =
// tokens x choices, tiles <= pairs / 16 + experts), so a step neither waits for the routing nor
// changes its launches with it: a captured step replays for any routing.
//
//   kvc_moe_route    scores = softmax(logits) or sigmoid(logits) in float32; the choice is made on the
//                    scores plus an optional correction per expert: the `keep` groups that are worth
//                    most (a group's best choice score, or the sum of its best two); the `top` best
//                    experts of those groups (the lower index on a tie); weights = the chosen experts'
//                    plain scores / (their sum + 1e-20) * weight_scale.  A wave a token.
//   kvc_moe_router   the router's product (float32 sums in one fixed order over rows of either dtype)
//                    and the choice in one kernel.
//   kvc_moe_align    pairs sorted by expert: sorted[i] = pair index (token * top + choice), and a
//                    list of tiles of up to 16 (or 64) sorted rows that belong to one expert each.
//   kvc_moe_gemm     for every tile, rows x that expert's matrix.  Gated: gate and up rows of the
//                    expert side by side in one pass, and the activation
//                    min(g, limit) * sigmoid(alpha * g) * (clamp(u, -limit, limit) + up_shift) on the way
//                    out (an infinite limit, alpha 1 and up_shift 0: silu(g) * u).
//                    bfloat16 operands go through the matrix cores (16 x 16 x 32, the expert's rows as
//                    the A operand, the tokens as B) with float32 sums; float32 operands, and rows
//                    that 16-byte loads do not divide, are summed in float32 in index order.  A row's sums do not depend on which tile it is in.
//   kvc_moe_combine  out[t] = sum_c weight[t, c] * y[t * top + c] (+ up to two more row sets),
//                    float32, in the order of the choices; or added into out (the residual stream).
//   kvc_clamped_glu  the same activation for a feed-forward that every token runs.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "gemm_common.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

#define S(stream) reinterpret_cast<hipStream_t>(stream)

constexpr int kTileRows = 16;
constexpr int kBigTileRows = 64;

__device__ __forceinline__ float clamped_glu(float g, float u, float limit, float alpha, float shift) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + shift);
}

// the lane that holds the largest value (the lowest index among equals) tells everyone
__device__ __forceinline__ void wave_argmax(float& val, int& idx) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(val, o, kWave);
    const int oi = __shfl_xor(idx, o, kWave);
    if (ov > val || (ov == val && oi < idx)) {
      val = ov;
      idx = oi;
    }
  }
}

// How a token's experts are chosen from its logits.  score_fn 0: softmax over the experts, 1: a
// sigmoid of each logit.  The choice is made on score + correction[e] (correction may be null) and
// may so be negative; the weights are the plain scores of the chosen, over their sum (+ 1e-20),
// times weight_scale.  With keep < groups only the experts of the best `keep` of `groups` equal
// groups of neighbours may be chosen; a group is worth the sum of its `group_best` (1 or 2) largest
// choice scores.  The lower index wins a tie.
struct RouteRule {
  int top, groups, keep, score_fn, group_best;
  const float* correction;
  float weight_scale;
};

// One token's choice by one wave: z [E] logits (global or LDS), sc [E], pk [E] and gs [groups] LDS
// scratch (sc may be z itself).
__device__ __forceinline__ void route_one(int32_t* __restrict__ choice, float* __restrict__ weight, const float* z,
                                          float* sc, float* pk, float* gs, int lane, int E, const RouteRule& rule) {
  const int top = rule.top, groups = rule.groups, keep = rule.keep;
  if (rule.score_fn == 0) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += kWave) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += kWave) {
      const float p = expf(z[e] - mx);
      sc[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int e = lane; e < E; e += kWave) sc[e] *= inv;
  } else {
    for (int e = lane; e < E; e += kWave) sc[e] = 1.f / (1.f + expf(-z[e]));
  }
  for (int e = lane; e < E; e += kWave) pk[e] = sc[e] + (rule.correction != nullptr ? rule.correction[e] : 0.f);
  __builtin_amdgcn_wave_barrier();
  const int per = E / groups;
  if (keep < groups) {
    for (int g = lane; g < groups; g += kWave) {
      float best = -INFINITY, second = -INFINITY;
      for (int i = 0; i < per; ++i) {
        const float s = pk[g * per + i];
        if (s > best) {
          second = best;
          best = s;
        } else if (s > second) {
          second = s;
        }
      }
      gs[g] = (rule.group_best >= 2 && per >= 2) ? best + second : best;
    }
    __builtin_amdgcn_wave_barrier();
    // the best `keep` groups are marked with +inf; the others' experts are taken out
    for (int r = 0; r < keep; ++r) {
      float val = -INFINITY;
      int idx = 0x7fffffff;
      for (int g = lane; g < groups; g += kWave) {
        const float s = gs[g];
        if (s != INFINITY && (s > val || (s == val && g < idx))) {
          val = s;
          idx = g;
        }
      }
      wave_argmax(val, idx);
      if (lane == 0 && idx < groups) gs[idx] = INFINITY;
      __builtin_amdgcn_wave_barrier();
    }
    for (int e = lane; e < E; e += kWave)
      if (gs[e / per] != INFINITY) pk[e] = -INFINITY;  // choice scores may be negative: minus infinity, not zero
    __builtin_amdgcn_wave_barrier();
  }
  float total = 0.f;
  float mine = 0.f;  // lane c keeps the c-th choice's score
  int mine_idx = 0;
  for (int c = 0; c < top; ++c) {
    float val = -INFINITY;
    int idx = 0x7fffffff;
    for (int e = lane; e < E; e += kWave) {
      const float s = pk[e];
      if (s > val || (s == val && e < idx)) {
        val = s;
        idx = e;
      }
    }
    wave_argmax(val, idx);
    if (idx >= E) idx = 0;
    // fewer allowed experts than choices: a weight of zero
    const float plain = (val == -INFINITY) ? 0.f : sc[idx];
    total += plain;
    if (lane == c) {
      mine = plain;
      mine_idx = idx;
    }
    __builtin_amdgcn_wave_barrier();
    if (lane == 0) pk[idx] = -INFINITY;
    __builtin_amdgcn_wave_barrier();
  }
  const float norm = rule.weight_scale / (total + 1e-20f);
  if (lane < top) {
    choice[lane] = mine_idx;
    weight[lane] = mine * norm;
  }
}

__global__ __launch_bounds__(256) void moe_route_kernel(int32_t* __restrict__ choice, float* __restrict__ weight,
                                                        const float* __restrict__ logits, int T, int E,
                                                        RouteRule rule) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  float* sc = lds + wave * (2 * E + rule.groups);  // scores, choice scores, then the groups' worth
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;  // the whole wave
  route_one(choice + static_cast<int64_t>(t) * rule.top, weight + static_cast<int64_t>(t) * rule.top,
            logits + static_cast<int64_t>(t) * E, sc, sc + E, sc + 2 * E, lane, E, rule);
}

// The router whole: logits = x W^T in float32 (x of either dtype, its values as they are), then the
// choice as in moe_route_kernel.  A block takes TOK tokens.  Its four waves share K: lane l of wave
// w sums the products of the values 4 l .. 4 l + 3 of the pieces of 256 that are the wave's (every
// fourth piece) for each of up to 32 experts at a time (a fetched piece of the router's row meets all
// TOK tokens); the 256 partial sums of a logit are added in wave and lane order through LDS: one
// fixed order, whatever the batch.  The first wave then chooses.
template <typename T, int TOK>
__global__ __launch_bounds__(256) void moe_router_kernel(int32_t* __restrict__ choice, float* __restrict__ weight,
                                                         const T* __restrict__ x, int64_t x_stride,
                                                         const float* __restrict__ wr, int T_, int H, int E,
                                                         RouteRule rule, int vectors) {
  constexpr int EB = 32, PR = EB + 1;
  extern __shared__ float lds[];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  float* part = lds;                       // [256][EB + 1]
  float* z = lds + 256 * PR;               // [TOK][2 E + groups]
  const int zrow = 2 * E + rule.groups;
  const int t0 = blockIdx.x * TOK;
  for (int e0 = 0; e0 < E; e0 += EB) {
    const int ne = (E - e0 < EB) ? E - e0 : EB;
    float acc[TOK][EB];
#pragma unroll
    for (int j = 0; j < TOK; ++j)
#pragma unroll
      for (int e = 0; e < EB; ++e) acc[j][e] = 0.f;
    for (int k = 4 * lane + 4 * kWave * wave; k < H; k += 16 * kWave) {
      float xv[TOK][4];
#pragma unroll
      for (int j = 0; j < TOK; ++j) {
        const T* xr = x + static_cast<int64_t>(t0 + j < T_ ? t0 + j : t0) * x_stride + k;
#pragma unroll
        for (int i = 0; i < 4; ++i) xv[j][i] = (k + i < H) ? to_float(xr[i]) : 0.f;
      }
      // every expert's piece is asked for before any is used, with no branch between the loads
      // (an expert beyond the last reads the last one's row again; its sums are dropped)
      float wv[EB][4];
#pragma unroll
      for (int e = 0; e < EB; ++e) {
        const float* wp = wr + static_cast<int64_t>(e < ne ? e0 + e : E - 1) * H + k;
        if (vectors) {
          const float4 v4 = *reinterpret_cast<const float4*>(wp);
          wv[e][0] = v4.x; wv[e][1] = v4.y; wv[e][2] = v4.z; wv[e][3] = v4.w;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) wv[e][i] = (k + i < H) ? wp[i] : 0.f;
        }
      }
#pragma unroll
      for (int e = 0; e < EB; ++e)
#pragma unroll
        for (int j = 0; j < TOK; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[j][e] = fmaf(xv[j][i], wv[e][i], acc[j][e]);
    }
#pragma unroll
    for (int j = 0; j < TOK; ++j) {
      __syncthreads();  // the partial sums of the token before have been added up
#pragma unroll
      for (int e = 0; e < EB; ++e) part[threadIdx.x * PR + e] = acc[j][e];
      __syncthreads();
      if (threadIdx.x < ne) {
        float sum = 0.f;
        for (int l = 0; l < 256; ++l) sum += part[l * PR + threadIdx.x];
        z[j * zrow + e0 + threadIdx.x] = sum;
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
  for (int j = 0; j < TOK; ++j) {
    const int t = t0 + j;
    if (t >= T_) break;  // the whole wave
    float* zr = z + j * zrow;
    route_one(choice + static_cast<int64_t>(t) * rule.top, weight + static_cast<int64_t>(t) * rule.top, zr, zr, zr + E,
              zr + 2 * E, lane, E, rule);
  }
}

// One block.  counts -> offsets -> sorted pairs -> tiles.
__global__ __launch_bounds__(1024) void moe_align_kernel(int32_t* __restrict__ sorted, int32_t* __restrict__ tiles,
                                                         int32_t* __restrict__ num_tiles,
                                                         const int32_t* __restrict__ choice, int pairs, int E,
                                                         int max_tiles, int tile_rows) {
  extern __shared__ int32_t ilds[];
  int32_t* count = ilds;           // [E]
  int32_t* offset = count + E;     // [E + 1]
  int32_t* cursor = offset + E + 1;  // [E]
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = choice[i];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      offset[e] = at;
      cursor[e] = 0;
      for (int r = 0; r < count[e] && nt < max_tiles; r += tile_rows, ++nt) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = at + r;
        tiles[3 * nt + 2] = (count[e] - r < tile_rows) ? count[e] - r : tile_rows;
      }
      at += count[e];
    }
    offset[E] = at;
    *num_tiles = nt;
  }
  __syncthreads();
  // an expert's pairs take their places in the order in which their threads arrive: a row's sums
  // do not depend on its place
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = choice[i];
    if (e < 0 || e >= E) continue;
    const int place = atomicAdd(&cursor[e], 1);
    sorted[offset[e] + place] = i;
  }
}

// bfloat16: a block of four waves takes one tile of rows and 64 columns (16 a wave).  A pass covers
// 64 values along K: lane (li, lk) fetches the 16 values from 16 lk of its weight row and of its
// token row (32 contiguous bytes, so that the four lanes of a row read one 128-byte line) and the two
// matrix instructions of the pass take its first and its second eight (both operands are dealt the
// same way, so each product still sums over all of K); the values of the next two passes are asked for
// before this pass's products.
template <int GATED, typename TO, int PACKED>
__global__ __launch_bounds__(256) void moe_gemm_bf16_kernel(
    TO* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ x, int64_t x_stride,
    const bf16_t* __restrict__ w, const int32_t* __restrict__ sorted, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ num_tiles, int N, int K, int in_div, int out_sorted, float limit, float alpha, float shift) {
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;
  const int e = tiles[3 * tile], r0 = tiles[3 * tile + 1], nr = tiles[3 * tile + 2];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int n0 = (blockIdx.y * 4 + wave) * 16;
  if (n0 >= N) return;
  const int li = lane & 15, lk = lane >> 4;
  // B operand: token row li of the tile; A operand: the expert's row n0 + li
  const bool row_ok = li < nr;
  const int pair = sorted[r0 + (row_ok ? li : 0)];
  const int64_t in_row = in_div > 0 ? pair / in_div : r0 + (row_ok ? li : 0);
  // PACKED: w is the copy that `kvc_pack_weight` makes, tiles of 16 rows x 32 values of K in one
  // piece of 1 KB each, so a wave's load of an operand is one contiguous kilobyte instead of 128 bytes
  // from each of 16 rows that lie 2 K bytes apart (which meet in the same memory channels); the lanes
  // then take K in the plain order, 8 values from 8 lk of each 32.
  const bf16_t* xr = x + in_row * x_stride + (PACKED ? 8 : 16) * lk;
  const int wrow = n0 + li < N ? n0 + li : N - 1;
  const int64_t rows_per_expert = GATED ? 2 * static_cast<int64_t>(N) : N;
  const bf16_t* wr = PACKED ? w + ((static_cast<int64_t>(e) * rows_per_expert + n0) >> 4) * (K / 32) * 512 + li * 32 + lk * 8
                            : w + (static_cast<int64_t>(e) * rows_per_expert + wrow) * K + 16 * lk;
  const bf16_t* wr2 = wr + static_cast<int64_t>(N) * K;  // the up rows follow the gate rows (in either order of storage)
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
  const int k_main = K & ~63;
  // two passes are on their way while one is multiplied
  bf16x8_t an[2][2], a2n[2][2], bn[2][2];
  auto fetch = [&](int k, int slot) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int64_t wo = PACKED ? static_cast<int64_t>(k / 32 + h) * 512 : k + 8 * h;
      an[slot][h] = *reinterpret_cast<const bf16x8_t*>(wr + wo);
      if (GATED) a2n[slot][h] = *reinterpret_cast<const bf16x8_t*>(wr2 + wo);
      // a row that is not there reads the tile's first
      bn[slot][h] = *reinterpret_cast<const bf16x8_t*>(xr + k + (PACKED ? 32 : 8) * h);
    }
  };
  if (k_main > 0) fetch(0, 0);
  if (k_main > 64) fetch(64, 1);
  for (int k = 0; k < k_main; k += 128) {
    // slot 0 holds pass k, slot 1 pass k + 64; each is asked for again as soon as it has been used
    bf16x8_t a0[2], a20[2], b0[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      a0[h] = an[0][h];
      if (GATED) a20[h] = a2n[0][h];
      b0[h] = row_ok ? bn[0][h] : zero8();
    }
    if (k + 128 < k_main) fetch(k + 128, 0);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[h], b0[h], acc, 0, 0, 0);
      if (GATED) acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a20[h], b0[h], acc2, 0, 0, 0);
    }
    if (k + 64 < k_main) {
      bf16x8_t a1[2], a21[2], b1[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        a1[h] = an[1][h];
        if (GATED) a21[h] = a2n[1][h];
        b1[h] = row_ok ? bn[1][h] : zero8();
      }
      if (k + 192 < k_main) fetch(k + 192, 1);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[h], b1[h], acc, 0, 0, 0);
        if (GATED) acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a21[h], b1[h], acc2, 0, 0, 0);
      }
    }
  }
  if (k_main < K) {  // a ragged end along K (a multiple of 8): element by element, zeros beyond
    bf16x8_t a[2], a2[2], b[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      a[h] = zero8(); a2[h] = zero8(); b[h] = zero8();
      for (int i = 0; i < 8; ++i) {
        const int off = k_main + 8 * h + i;  // from the lane's own start 16 lk
        if (off + 16 * lk < K) {
          a[h][i] = reinterpret_cast<const __bf16*>(wr)[off];
          if (GATED) a2[h][i] = reinterpret_cast<const __bf16*>(wr2)[off];
          if (row_ok) b[h][i] = reinterpret_cast<const __bf16*>(xr)[off];
        }
      }
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[h], b[h], acc, 0, 0, 0);
      if (GATED) acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[h], b[h], acc2, 0, 0, 0);
    }
  }
  // lane holds column (token) li, rows (features) n0 + 4 * lk + i
  if (!row_ok) return;
  if (GATED) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = clamped_glu(acc[i], acc2[i], limit, alpha, shift);
  }
  const int64_t out_row = out_sorted ? r0 + li : pair;
  const int nf = n0 + 4 * lk;
  if (nf < N) store4<TO>(out + out_row * out_stride + nf, acc, N - nf);
}

// bfloat16, tiles of 64 rows: a block of four waves takes the tile's rows and 128 columns (gated;
// 256 otherwise).  The rows' chunk of 64 values along K goes through LDS, which all waves read as
// the B operand (four row blocks of 16); every wave fetches the weight rows of its own columns
// straight into registers as the A operand (NF blocks of 16 columns, for gate and for up), one
// chunk ahead of the products.  Every fetched weight meets 64 rows, every row 128 or 256 columns.
template <int GATED, typename TO, int PACKED>
__global__ __launch_bounds__(256) void moe_gemm_tiled_kernel(
    TO* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ x, int64_t x_stride,
    const bf16_t* __restrict__ w, const int32_t* __restrict__ sorted, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ num_tiles, int N, int K, int in_div, int out_sorted, float limit, float alpha, float shift) {
  constexpr int NF = GATED ? 2 : 4;   // column blocks of 16 a wave
  constexpr int NR = kBigTileRows / 16;
  constexpr int KC = 64;              // values of K a pass (two matrix instructions deep)
  constexpr int KROW = KC + 8;        // a row's chunk in LDS, padded against bank conflicts
  __shared__ __attribute__((aligned(16))) bf16_t x_s[kBigTileRows * KROW];
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;
  const int e = tiles[3 * tile], r0 = tiles[3 * tile + 1], nr = tiles[3 * tile + 2];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int li = lane & 15, lk = lane >> 4;
  const int n0 = (blockIdx.y * 4 + wave) * 16 * NF;
  const bool wave_live = n0 < N;  // the same for the whole wave
  // staging: thread t brings 16 values of row t / 4 of the tile
  const int srow = threadIdx.x >> 2, spart = threadIdx.x & 3;
  const bool srow_ok = srow < nr;
  const int srow_safe = srow_ok ? srow : 0;  // a row that is not there reads the tile's first, and is set to zero
  const int64_t in_row = in_div > 0 ? sorted[r0 + srow_safe] / in_div : r0 + srow_safe;
  const bf16_t* xp = x + in_row * x_stride + 16 * spart;
  const int64_t rows_per_expert = GATED ? 2 * static_cast<int64_t>(N) : N;
  const bf16_t* wp[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int wrow = n0 + 16 * f + li < N ? n0 + 16 * f + li : N - 1;
    // PACKED (N a multiple of 16): the copy in pieces of 16 rows x 32 values, one contiguous kilobyte a load
    const int ntile = n0 + 16 * f < N ? n0 + 16 * f : N - 16;
    wp[f] = PACKED ? w + ((static_cast<int64_t>(e) * rows_per_expert + ntile) >> 4) * (K / 32) * 512 + li * 32 + lk * 8
                   : w + (static_cast<int64_t>(e) * rows_per_expert + wrow) * K + 8 * lk;
  }
  const int64_t up_off = static_cast<int64_t>(N) * K;
  f32x4_t acc[NF][NR], acc2[GATED ? NF : 1][NR];
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      acc[f][r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (GATED) acc2[f][r] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  uint4 x_next[2] = {uint4{0u, 0u, 0u, 0u}, uint4{0u, 0u, 0u, 0u}};
  bf16x8_t w_next[2][NF], w2_next[2][GATED ? NF : 1];
  // a pass's second half may lie beyond K (K a multiple of 32 only): it then reads the first half
  // again and is not multiplied
  auto fetch = [&](int k) {
    const bool two = k + 32 < K;
    const int c0 = (two || spart < 2) ? 0 : -16 * spart;  // columns beyond K read the pass's first instead
    x_next[0] = *reinterpret_cast<const uint4*>(xp + k + c0);
    x_next[1] = *reinterpret_cast<const uint4*>(xp + k + c0 + 8);
    if (wave_live) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int kk = k + ((h && two) ? 32 : 0);
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          const int64_t wo = PACKED ? static_cast<int64_t>(kk / 32) * 512 : kk;
          w_next[h][f] = *reinterpret_cast<const bf16x8_t*>(wp[f] + wo);
          if (GATED) w2_next[h][f] = *reinterpret_cast<const bf16x8_t*>(wp[f] + up_off + wo);
        }
      }
    }
  };
  fetch(0);
  for (int k = 0; k < K; k += KC) {
    const bool two = k + 32 < K;
    __syncthreads();  // the chunk before has been read by every wave
    // thread t's 16 values: columns 16 spart .. of the pass; K shorter than a whole pass leaves zeros
    const bool keep = srow_ok && (two || spart < 2);
    *reinterpret_cast<uint4*>(x_s + srow * KROW + 16 * spart) = keep ? x_next[0] : uint4{0u, 0u, 0u, 0u};
    *reinterpret_cast<uint4*>(x_s + srow * KROW + 16 * spart + 8) = keep ? x_next[1] : uint4{0u, 0u, 0u, 0u};
    bf16x8_t wa[2][NF], wa2[2][GATED ? NF : 1];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        wa[h][f] = w_next[h][f];
        if (GATED) wa2[h][f] = w2_next[h][f];
      }
    if (k + KC < K) fetch(k + KC);
    __syncthreads();
    if (wave_live) {  // scalar: matrix instructions are skipped by a branch, never by a lane mask
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if (h == 1 && !two) break;  // scalar
#pragma unroll
        for (int r = 0; r < NR; ++r) {
          const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(x_s + (16 * r + li) * KROW + 32 * h + 8 * lk);
#pragma unroll
          for (int f = 0; f < NF; ++f) {
            acc[f][r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[h][f], b, acc[f][r], 0, 0, 0);
            if (GATED) acc2[f][r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa2[h][f], b, acc2[f][r], 0, 0, 0);
          }
        }
      }
    }
  }
  if (!wave_live) return;
  // lane holds row 16 r + li of the tile, columns n0 + 16 f + 4 lk + i
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int row = 16 * r + li;
    if (row >= nr) continue;
    const int64_t out_row = out_sorted ? r0 + row : sorted[r0 + row];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      f32x4_t v = acc[f][r];
      if (GATED) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = clamped_glu(v[i], acc2[f][r][i], limit, alpha, shift);
      }
      const int nf = n0 + 16 * f + 4 * lk;
      if (nf < N) store4<TO>(out + out_row * out_stride + nf, v, N - nf);
    }
  }
}

// Any operand type and any sizes: a thread a (row, column) pair of the tile, float32 sums in index
// order.  The float32 path, and bfloat16 rows that 16-byte loads do not divide.
template <int GATED, typename TI, typename TO>
__global__ __launch_bounds__(256) void moe_gemm_plain_kernel(
    TO* __restrict__ out, int64_t out_stride, const TI* __restrict__ x, int64_t x_stride,
    const TI* __restrict__ w, const int32_t* __restrict__ sorted, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ num_tiles, int N, int K, int in_div, int out_sorted, float limit, float alpha, float shift) {
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;
  const int e = tiles[3 * tile], r0 = tiles[3 * tile + 1], nr = tiles[3 * tile + 2];
  const int li = threadIdx.x & 15, col = threadIdx.x >> 4;  // 16 rows x 16 columns a pass
  if (li >= nr) return;
  const int pair = sorted[r0 + li];
  const int64_t in_row = in_div > 0 ? pair / in_div : r0 + li;
  const TI* xr = x + in_row * x_stride;
  const int64_t rows_per_expert = GATED ? 2 * static_cast<int64_t>(N) : N;
  const int64_t out_row = out_sorted ? r0 + li : pair;
  for (int n = blockIdx.y * 64 + col; n < N && n < (blockIdx.y + 1) * 64; n += 16) {
    const TI* wr = w + (static_cast<int64_t>(e) * rows_per_expert + n) * K;
    float acc = 0.f, acc2 = 0.f;
    for (int k = 0; k < K; ++k) {
      const float xv = to_float(xr[k]);
      acc = fmaf(xv, to_float(wr[k]), acc);
      if (GATED) acc2 = fmaf(xv, to_float(wr[static_cast<int64_t>(N) * K + k]), acc2);
    }
    out[out_row * out_stride + n] = from_float<TO>(GATED ? clamped_glu(acc, acc2, limit, alpha, shift) : acc);
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y,
                                                          const float* __restrict__ weight, int top,
                                                          const TA* __restrict__ add0, const float* __restrict__ add1,
                                                          int T, int H, int accumulate) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= static_cast<int64_t>(T) * H) return;
  const int t = static_cast<int>(idx / H), c = static_cast<int>(idx - static_cast<int64_t>(t) * H);
  float acc = 0.f;
  for (int j = 0; j < top; ++j)
    acc = fmaf(weight[static_cast<int64_t>(t) * top + j], y[(static_cast<int64_t>(t) * top + j) * H + c], acc);
  if (add0 != nullptr) acc += to_float(add0[idx]);
  if (add1 != nullptr) acc += add1[idx];
  out[idx] = accumulate ? out[idx] + acc : acc;
}

template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(T* __restrict__ out, const T* __restrict__ gate_up,
                                                          int64_t n, int I, float limit, float alpha, float shift) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t t = idx / I, i = idx - t * I;
  const T* row = gate_up + t * 2 * I;
  out[idx] = from_float<T>(clamped_glu(to_float(row[i]), to_float(row[I + i]), limit, alpha, shift));
}

}  // namespace

extern "C" int kvc_moe_route(int32_t* choice, float* weight, const float* logits, int T, int E, int top,
                             int groups, int keep, int score_fn, const float* correction, int group_best,
                             float weight_scale, kvc_stream stream) {
  if (T < 0 || E <= 0 || top <= 0 || top > E || top > kWave || groups <= 0 || E % groups || keep <= 0 ||
      keep > groups)
    return kvc_fail("kvc_moe_route: bad sizes (at most 64 choices; the experts in equal groups)");
  if ((score_fn != 0 && score_fn != 1) || (group_best != 1 && group_best != 2))
    return kvc_fail("kvc_moe_route: scores by softmax (0) or sigmoid (1); a group is worth its best 1 or 2");
  const RouteRule rule{top, groups, keep, score_fn, group_best, correction, weight_scale};
  const size_t lds = sizeof(float) * 4 * (2 * E + groups);
  if (lds > 60000) return kvc_fail("kvc_moe_route: too many experts for a wave's scores in LDS");
  if (T == 0) return 0;
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), lds, S(stream), choice, weight, logits, T, E,
                     rule);
  return kvc_check_launch("kvc_moe_route");
}

extern "C" int kvc_moe_router(int32_t* choice, float* weight, const void* x, int64_t x_stride, int x_dtype,
                              const float* router, int T, int H, int E, int top, int groups, int keep,
                              int score_fn, const float* correction, int group_best, float weight_scale,
                              kvc_stream stream) {
  if (T < 0 || H <= 0 || E <= 0 || top <= 0 || top > E || top > kWave || groups <= 0 || E % groups || keep <= 0 ||
      keep > groups || x_stride < H)
    return kvc_fail("kvc_moe_router: bad sizes (at most 64 choices; the experts in equal groups)");
  if ((score_fn != 0 && score_fn != 1) || (group_best != 1 && group_best != 2))
    return kvc_fail("kvc_moe_router: scores by softmax (0) or sigmoid (1); a group is worth its best 1 or 2");
  const RouteRule rule{top, groups, keep, score_fn, group_best, correction, weight_scale};
  if (T == 0) return 0;
  // four tokens a block where the blocks then still fill the chip several times over, else one
  const bool big = T >= 4 * 8 * kvc_device_compute_units();
  const int TOK = big ? 4 : 1;
  const size_t lds = sizeof(float) * (static_cast<size_t>(256) * 33 + static_cast<size_t>(TOK) * (2 * E + groups));
  if (lds > 160 * 1024) return kvc_fail("kvc_moe_router: too many experts for a block's LDS");
  const dim3 grid((T + TOK - 1) / TOK);
  // 16-byte loads of the router's rows where the rows allow
  const int vectors = H % 4 == 0 && (reinterpret_cast<uintptr_t>(router) & 15) == 0;
#define KVC_ROUTER(Tp, TOK_)                                                                                    \
  do {                                                                                                          \
    if (lds > 64 * 1024) {                                                                                      \
      const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_router_kernel<Tp, TOK_>),  \
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
      if (attr != hipSuccess) return kvc_fail("kvc_moe_router: the kernel's LDS size was refused");            \
    }                                                                                                           \
    hipLaunchKernelGGL((moe_router_kernel<Tp, TOK_>), grid, dim3(256), lds, S(stream), choice, weight,          \
                       static_cast<const Tp*>(x), x_stride, router, T, H, E, rule, vectors);             \
  } while (0)
  if (x_dtype == 1 && big) KVC_ROUTER(bf16_t, 4);
  else if (x_dtype == 1) KVC_ROUTER(bf16_t, 1);
  else if (x_dtype == 0 && big) KVC_ROUTER(float, 4);
  else if (x_dtype == 0) KVC_ROUTER(float, 1);
  else return kvc_fail("kvc_moe_router: unknown dtype code");
#undef KVC_ROUTER
  return kvc_check_launch("kvc_moe_router");
}

extern "C" int kvc_moe_max_tiles(int pairs, int E, int tile_rows) {
  return (pairs + tile_rows - 1) / tile_rows + E;
}

// Tiles of 64 rows where the experts have that many rows on average (portions of prompts): the
// tiled kernel then uses every fetched weight four times as often; tiles of 16 otherwise.
extern "C" int kvc_moe_tile_rows(int pairs, int E) { return pairs >= 64 * E ? kBigTileRows : kTileRows; }

extern "C" int kvc_moe_align(int32_t* sorted, int32_t* tiles, int32_t* num_tiles, const int32_t* choice,
                             int pairs, int E, int max_tiles, int tile_rows, kvc_stream stream) {
  if (tile_rows != kTileRows && tile_rows != kBigTileRows) return kvc_fail("kvc_moe_align: tiles of 16 or 64 rows");
  if (pairs < 0 || E <= 0 || max_tiles < kvc_moe_max_tiles(pairs, E, tile_rows))
    return kvc_fail("kvc_moe_align: bad sizes, or room for fewer tiles than the routing may need");
  const size_t lds = sizeof(int32_t) * (3 * E + 1);
  if (lds > 60000) return kvc_fail("kvc_moe_align: too many experts");
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), lds, S(stream), sorted, tiles, num_tiles, choice,
                     pairs, E, max_tiles, tile_rows);
  return kvc_check_launch("kvc_moe_align");
}

extern "C" int kvc_moe_gemm(void* out, int64_t out_stride, int out_dtype, const void* x, int64_t x_stride,
                            const void* w, int dtype, const int32_t* sorted, const int32_t* tiles,
                            const int32_t* num_tiles, int max_tiles, int tile_rows, int N, int K, int in_div,
                            int out_sorted, int gated, float limit, float alpha, float up_shift, int packed,
                            kvc_stream stream) {
  if (max_tiles < 0 || N <= 0 || K <= 0 || x_stride < K || out_stride < N)
    return kvc_fail("kvc_moe_gemm: bad sizes");
  if (tile_rows != kTileRows && tile_rows != kBigTileRows) return kvc_fail("kvc_moe_gemm: tiles of 16 or 64 rows");
  if (max_tiles == 0) return 0;
  dim3 grid(max_tiles, (N + 63) / 64);
  if (grid.y > 65535u) return kvc_fail("kvc_moe_gemm: too many columns");
#define KVC_MOE_ARGS sorted, tiles, num_tiles, N, K, in_div, out_sorted, limit, alpha, up_shift
#define KVC_MOE_LAUNCH(KERNEL, TI, TO)                                                                          \
  hipLaunchKernelGGL(KERNEL, grid, dim3(256), 0, S(stream), static_cast<TO*>(out), out_stride,                   \
                     static_cast<const TI*>(x), x_stride, static_cast<const TI*>(w), KVC_MOE_ARGS)
  if (out_dtype != 0 && out_dtype != 1) return kvc_fail("kvc_moe_gemm: unknown dtype code");
  if (dtype == 1) {
    // the matrix cores read 16 bytes at a time: rows of a multiple of 8 values, 16-byte aligned
    const bool vectors = K % 8 == 0 && x_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(w) & 15) == 0;
    if (tile_rows == kBigTileRows) {
      if (!vectors || K % 32) return kvc_fail("kvc_moe_gemm: tiles of 64 rows need K to be a multiple of 32");
      if (packed && (N % 16 || K % 64))
        return kvc_fail("kvc_moe_gemm: a packed matrix has experts of a multiple of 16 rows of a multiple of 64");
      grid.y = gated ? (N + 127) / 128 : (N + 255) / 256;
      if (packed) {
        if (gated && out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<1, bf16_t, 1>), bf16_t, bf16_t);
        else if (gated) KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<1, float, 1>), bf16_t, float);
        else if (out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<0, bf16_t, 1>), bf16_t, bf16_t);
        else KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<0, float, 1>), bf16_t, float);
      } else {
        if (gated && out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<1, bf16_t, 0>), bf16_t, bf16_t);
        else if (gated) KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<1, float, 0>), bf16_t, float);
        else if (out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<0, bf16_t, 0>), bf16_t, bf16_t);
        else KVC_MOE_LAUNCH((moe_gemm_tiled_kernel<0, float, 0>), bf16_t, float);
      }
    } else if (packed) {
      if (!vectors || N % 16 || K % 64)
        return kvc_fail("kvc_moe_gemm: a packed matrix has experts of a multiple of 16 rows of a multiple of 64");
      if (gated && out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<1, bf16_t, 1>), bf16_t, bf16_t);
      else if (gated) KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<1, float, 1>), bf16_t, float);
      else if (out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<0, bf16_t, 1>), bf16_t, bf16_t);
      else KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<0, float, 1>), bf16_t, float);
    } else if (vectors) {
      if (gated && out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<1, bf16_t, 0>), bf16_t, bf16_t);
      else if (gated) KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<1, float, 0>), bf16_t, float);
      else if (out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<0, bf16_t, 0>), bf16_t, bf16_t);
      else KVC_MOE_LAUNCH((moe_gemm_bf16_kernel<0, float, 0>), bf16_t, float);
    } else {
      if (gated && out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_plain_kernel<1, bf16_t, bf16_t>), bf16_t, bf16_t);
      else if (gated) KVC_MOE_LAUNCH((moe_gemm_plain_kernel<1, bf16_t, float>), bf16_t, float);
      else if (out_dtype == 1) KVC_MOE_LAUNCH((moe_gemm_plain_kernel<0, bf16_t, bf16_t>), bf16_t, bf16_t);
      else KVC_MOE_LAUNCH((moe_gemm_plain_kernel<0, bf16_t, float>), bf16_t, float);
    }
  } else if (dtype == 0) {
    if (out_dtype != 0) return kvc_fail("kvc_moe_gemm: float32 operands give float32 rows");
    if (tile_rows != kTileRows || packed) return kvc_fail("kvc_moe_gemm: float32 operands take tiles of 16 rows of a row-major matrix");
    if (gated) KVC_MOE_LAUNCH((moe_gemm_plain_kernel<1, float, float>), float, float);
    else KVC_MOE_LAUNCH((moe_gemm_plain_kernel<0, float, float>), float, float);
  } else {
    return kvc_fail("kvc_moe_gemm: unknown dtype code");
  }
#undef KVC_MOE_LAUNCH
#undef KVC_MOE_ARGS
  return kvc_check_launch("kvc_moe_gemm");
}

extern "C" int kvc_moe_combine(float* out, const float* y, const float* weight, int top, const void* add0,
                               int add0_dtype, const float* add1, int T, int H, int accumulate,
                               kvc_stream stream) {
  if (T < 0 || H <= 0 || top < 0) return kvc_fail("kvc_moe_combine: bad sizes");
  if (T == 0) return 0;
  const int64_t n = static_cast<int64_t>(T) * H;
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  if (add0_dtype == 1) {
    hipLaunchKernelGGL((moe_combine_kernel<bf16_t>), grid, dim3(256), 0, S(stream), out, y, weight, top,
                       static_cast<const bf16_t*>(add0), add1, T, H, accumulate);
  } else {
    hipLaunchKernelGGL((moe_combine_kernel<float>), grid, dim3(256), 0, S(stream), out, y, weight, top,
                       static_cast<const float*>(add0), add1, T, H, accumulate);
  }
  return kvc_check_launch("kvc_moe_combine");
}

extern "C" int kvc_clamped_glu(void* out, const void* gate_up, int T, int I, float limit, float alpha, int dtype,
                               kvc_stream stream) {
  if (T < 0 || I <= 0) return kvc_fail("kvc_clamped_glu: bad sizes");
  if (T == 0) return 0;
  const int64_t n = static_cast<int64_t>(T) * I;
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL((clamped_glu_kernel<Tp>), grid, dim3(256), 0, S(stream),
                                        static_cast<Tp*>(out), static_cast<const Tp*>(gate_up), n, I, limit, alpha, 1.f));
  return kvc_check_launch("kvc_clamped_glu");
}
