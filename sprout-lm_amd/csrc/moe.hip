// Routing of a feed-forward with experts: choice of the experts, the order in which the grouped products walk
// the (token, choice) pairs, and the weighted sum of the experts' outputs.  Everything float32; nothing is
// decided on the host, so a step can be recorded into a graph.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

// The `top` largest of a token's `experts` logits (the lowest index wins a tie), in falling order, and the softmax
// over the chosen logits alone.
__device__ __forceinline__ void route_token(const float* __restrict__ z, int experts, int top, int32_t* __restrict__ id,
                                            float* __restrict__ w, bool sigmoid = false) {
  // the k-th choice is the largest logit that comes after the (k-1)-th in the order (falling value, rising index):
  // nothing already written is read back
  float prev_z = INFINITY, top_z = 0.f, sum = 0.f;
  int prev = -1;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float best_z = 0.f;
    for (int e = 0; e < experts; ++e) {
      const float v = z[e];
      const bool after = k == 0 || v < prev_z || (v == prev_z && e > prev);
      if (after && (best < 0 || v > best_z)) { best = e; best_z = v; }
    }
    if (best < 0) best = (prev + 1) % experts;      // only where logits are not numbers
    if (k == 0) top_z = best_z;
    const float ex = sigmoid ? 1.0f / (1.0f + expf(-best_z)) : expf(best_z - top_z);
    sum += ex;
    id[k] = best;
    w[k] = ex;
    prev = best;
    prev_z = best_z;
  }
  const float scale = sigmoid ? 1.0f : 1.0f / sum;
  for (int k = 0; k < top; ++k) w[k] *= scale;
}

// The same choice by a whole wave, for up to 256 experts: lane l holds the logits of experts l, l + 64, ..., one
// coalesced load, and every choice is a reduction over the wave (larger value first, lower index among equals).
constexpr int kWaveExperts = 256;
__device__ __forceinline__ void route_token_wave(const float* __restrict__ z, int experts, int top, int32_t* __restrict__ id,
                                                 float* __restrict__ w, int lane, bool sigmoid = false) {
  constexpr int J = kWaveExperts / 64, NONE = 0x7fffffff;
  float v[J];
  unsigned taken = 0;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int e = lane + 64 * j;
    v[j] = e < experts ? z[e] : 0.f;
    if (e >= experts) taken |= 1u << j;
  }
  int my_id[J];
  float my_ex[J], top_z = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = 0.f;
    int be = NONE;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (!((taken >> j) & 1) && (be == NONE || v[j] > bv)) { bv = v[j]; be = lane + 64 * j; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      if (oe != NONE && (be == NONE || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
    }
    if ((be & 63) == lane) taken |= 1u << (be >> 6);
    if (k == 0) top_z = bv;
    const float ex = sigmoid ? 1.0f / (1.0f + expf(-bv)) : expf(bv - top_z);
    sum += ex;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (k == lane + 64 * j) { my_id[j] = be; my_ex[j] = ex; }
  }
  const float scale = sigmoid ? 1.0f : 1.0f / sum;
#pragma unroll
  for (int j = 0; j < J; ++j)
    if (lane + 64 * j < top) { id[lane + 64 * j] = my_id[j]; w[lane + 64 * j] = my_ex[j] * scale; }
}

// How a token's experts are chosen and weighted.
//   mode 0: the `top` largest logits; weights = the softmax over the chosen logits alone.
//   mode 1: scores = the softmax over all outputs; the choice goes by score + correction[e], and only among the outputs
//           of the `keep` groups (of `groups` equal groups of neighbours) whose best such sum is largest; weights = the
//           chosen outputs' scores (without the correction) times `scale`, not renormalised.  Up to 256 outputs.
//   mode 2: the `top` largest logits; weights = the sigmoid of each chosen logit, not renormalised.
struct RouteRule {
  int mode;
  const float* correction;
  int groups, keep;
  float scale;
};

__device__ __forceinline__ void route_token_scored(const float* __restrict__ z, int outputs, int top, const RouteRule& rule,
                                                   int32_t* __restrict__ id, float* __restrict__ w, int lane) {
  constexpr int J = kWaveExperts / 64, NONE = 0x7fffffff;
  const int per = outputs / rule.groups;
  float score[J], choice[J];
  unsigned valid = 0, open = 0;
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int e = lane + 64 * j;
    score[j] = e < outputs ? z[e] : -INFINITY;
    if (e < outputs) valid |= 1u << j;
    mx = fmaxf(mx, score[j]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    score[j] = (valid >> j) & 1 ? expf(score[j] - mx) : 0.f;
    sum += score[j];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int j = 0; j < J; ++j) {
    score[j] = score[j] / sum;
    choice[j] = (valid >> j) & 1 ? score[j] + (rule.correction ? rule.correction[lane + 64 * j] : 0.f) : 0.f;
  }
  // the best groups, one at a time: the largest sum among the outputs of groups not yet opened names the next
  for (int r = 0; r < rule.keep; ++r) {
    float bv = 0.f;
    int be = NONE;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (((valid & ~open) >> j) & 1 && (be == NONE || choice[j] > bv)) { bv = choice[j]; be = lane + 64 * j; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      if (oe != NONE && (be == NONE || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
    }
    if (be == NONE) break;
    const int g = be / per;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if ((lane + 64 * j) / per == g) open |= (valid & (1u << j));
  }
  unsigned taken = ~open;
  int my_id[J];
  float my_w[J];
  for (int k = 0; k < top; ++k) {
    float bv = 0.f;
    int be = NONE;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (!((taken >> j) & 1) && (be == NONE || choice[j] > bv)) { bv = choice[j]; be = lane + 64 * j; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      if (oe != NONE && (be == NONE || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
    }
    if (be == NONE) be = k % outputs;      // only where too few outputs are open or logits are not numbers
    float mine = 0.f;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (j == (be >> 6)) mine = score[j];
    const float sv = __shfl(mine, be & 63, 64) * rule.scale;
    if ((be & 63) == lane) taken |= 1u << (be >> 6);
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (k == lane + 64 * j) { my_id[j] = be; my_w[j] = sv; }
  }
#pragma unroll
  for (int j = 0; j < J; ++j)
    if (lane + 64 * j < top) { id[lane + 64 * j] = my_id[j]; w[lane + 64 * j] = my_w[j]; }
}

// A wave a token (up to 256 experts), else a thread a token.
__global__ void route_topk_kernel(const float* __restrict__ logits, long long stride, int experts, int top,
                                  int32_t* __restrict__ ids, float* __restrict__ weights, int T, RouteRule rule) {
  if (experts <= kWaveExperts) {
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= T) return;
    if (rule.mode == 1) route_token_scored(logits + size_t(t) * stride, experts, top, rule, ids + size_t(t) * top, weights + size_t(t) * top, threadIdx.x & 63);
    else route_token_wave(logits + size_t(t) * stride, experts, top, ids + size_t(t) * top, weights + size_t(t) * top, threadIdx.x & 63,
                          rule.mode == 2);
    return;
  }
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  route_token(logits + size_t(t) * stride, experts, top, ids + size_t(t) * top, weights + size_t(t) * top, rule.mode == 2);
}

// One block: sorts the pairs (token, choice) by expert.  row_of_pair[p] = the row of pair p in the sorted order,
// pair_of_row its inverse; tiles [n][3] = (expert, first row, rows) cuts every expert's rows into tiles of at most
// tile_rows; *n_tiles = n.  Within an expert the rows of a wave's run of pairs stand together, in no
// fixed order (every row is computed for itself).  A wave owns a run of pairs and counts them in a row of LDS
// counters of its own (counts [waves][experts]), so an atomic meets at most the 63 other lanes of its instruction.
// With `logits` (and `weights`, `top`) the block first makes the choice itself (ids and weights are then outputs):
// choice and order in one launch.  Experts from `tiled` on get rows but no tiles: they have no weights to multiply
// (outputs that return their input), and the weighted sum treats their pairs by itself.
__global__ __launch_bounds__(1024) void route_sort_kernel(const float* __restrict__ logits, long long stride,
                                                          float* __restrict__ weights,
                                                          int top, int32_t* __restrict__ ids, int pairs, int experts,
                                                          int tiled, int tile_rows, int32_t* __restrict__ row_of_pair,
                                                          int32_t* __restrict__ pair_of_row, int32_t* __restrict__ tiles,
                                                          int32_t* __restrict__ n_tiles, RouteRule rule) {
  extern __shared__ int32_t lds[];      // [experts] first rows, then [waves][experts] counts
  const int waves = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int32_t* first = lds;
  int32_t* mine = lds + experts + wave * experts;
  for (int i = threadIdx.x; i < waves * experts; i += blockDim.x) lds[experts + i] = 0;
  if (logits) {
    if (rule.mode == 1)
      for (int t = wave; t < pairs / top; t += waves)
        route_token_scored(logits + size_t(t) * stride, experts, top, rule, ids + size_t(t) * top, weights + size_t(t) * top, lane);
    else if (experts <= kWaveExperts)
      for (int t = wave; t < pairs / top; t += waves)
        route_token_wave(logits + size_t(t) * stride, experts, top, ids + size_t(t) * top, weights + size_t(t) * top, lane,
                         rule.mode == 2);
    else
      for (int t = threadIdx.x; t < pairs / top; t += blockDim.x)
        route_token(logits + size_t(t) * stride, experts, top, ids + size_t(t) * top, weights + size_t(t) * top, rule.mode == 2);
  }
  __syncthreads();
  const int chunks = (pairs + 63) / 64, per_wave = (chunks + waves - 1) / waves;
  const int c_begin = min(chunks, wave * per_wave), c_end = min(chunks, c_begin + per_wave);
  for (int c = c_begin; c < c_end; ++c) {
    const int p = c * 64 + lane;
    if (p < pairs) atomicAdd(&mine[ids[p]], 1);      // the wave's own counters: only its 64 lanes ever meet there
  }
  __syncthreads();
  // per expert: where each wave's rows start within the expert, and the expert's total (left in wave 0's place)
  for (int e = threadIdx.x; e < experts; e += blockDim.x) {
    int running = 0;
    for (int w = 0; w < waves; ++w) {
      const int n = lds[experts + w * experts + e];
      lds[experts + w * experts + e] = running;
      running += n;
    }
    first[e] = running;      // for now the count
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int row = 0, n = 0;
    for (int e = 0; e < experts; ++e) {
      const int count = first[e];
      first[e] = row;
      for (int r = 0; r < count && e < tiled; r += tile_rows) {
        tiles[3 * n] = e;
        tiles[3 * n + 1] = row + r;
        tiles[3 * n + 2] = min(tile_rows, count - r);
        ++n;
      }
      row += count;
    }
    *n_tiles = n;
  }
  __syncthreads();
  for (int c = c_begin; c < c_end; ++c) {
    const int p = c * 64 + lane;
    if (p < pairs) {
      const int e = ids[p];
      const int row = first[e] + atomicAdd(&mine[e], 1);      // now the wave's next free row of the expert
      row_of_pair[p] = row;
      pair_of_row[row] = p;
    }
  }
}

// residual[t] += sum over the token's choices, in their order, of weight * (the expert's output row).  A block per
// token and 1,024 columns, a thread four neighbouring columns where rows are in fours.  With `ids` and `x`: a choice
// whose id is `real` or more has no output row; it stands for the token's own input row x[t] (of type TX).
template <typename TX>
__global__ __launch_bounds__(256) void route_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ row_of_pair,
                                                            const float* __restrict__ weights, int top,
                                                            float* __restrict__ residual, int H,
                                                            const int32_t* __restrict__ ids, const TX* __restrict__ x, int real) {
  const int t = blockIdx.x;
  const int32_t* rows = row_of_pair + size_t(t) * top;
  const float* wt = weights + size_t(t) * top;
  const int32_t* id = ids ? ids + size_t(t) * top : nullptr;
  const TX* own = ids ? x + size_t(t) * H : nullptr;
  if ((H & 3) == 0) {
    const int i = 4 * (blockIdx.y * 256 + threadIdx.x);
    if (i >= H) return;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < top; ++k) {
      const float w = weights ? wt[k] : 1.0f;
      float4 v;
      if (id && id[k] >= real) v = make_float4(to_float(own[i]), to_float(own[i + 1]), to_float(own[i + 2]), to_float(own[i + 3]));
      else v = *reinterpret_cast<const float4*>(y + size_t(rows[k]) * H + i);
      sum.x = fmaf(w, v.x, sum.x); sum.y = fmaf(w, v.y, sum.y); sum.z = fmaf(w, v.z, sum.z); sum.w = fmaf(w, v.w, sum.w);
    }
    float4* r = reinterpret_cast<float4*>(residual + size_t(t) * H + i);
    const float4 old = *r;
    *r = make_float4(old.x + sum.x, old.y + sum.y, old.z + sum.z, old.w + sum.w);
    return;
  }
  for (int i = blockIdx.y * 1024 + threadIdx.x; i < min(H, (int(blockIdx.y) + 1) * 1024); i += 256) {
    float sum = 0.f;
    for (int k = 0; k < top; ++k) sum = fmaf(weights ? wt[k] : 1.0f, id && id[k] >= real ? to_float(own[i]) : y[size_t(rows[k]) * H + i], sum);
    residual[size_t(t) * H + i] += sum;
  }
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_route_topk(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top) {
  SP_REQUIRE(T >= 0 && experts > 0 && top > 0 && top <= experts, "sp_route_topk: %d of %d experts", top, experts);
  SP_REQUIRE(logits && ids && weights, "sp_route_topk: null operand");
  if (T == 0) return 0;
  const int per_block = experts <= kWaveExperts ? 4 : 256;
  route_topk_kernel<<<(T + per_block - 1) / per_block, 256, 0, (hipStream_t)stream>>>(logits, experts, experts, top, ids, weights, T,
                                                                                      RouteRule{0, nullptr, 1, 1, 1.f});
  return check_launch("sp_route_topk");
}

extern "C" int sp_route_max_tiles(int pairs, int experts, int tile_rows) {
  // every expert's last tile may be a partial one
  return (pairs + tile_rows - 1) / tile_rows + (pairs < experts ? pairs : experts);
}

extern "C" int sp_route_sort(void* stream, const int32_t* ids, int pairs, int experts, int tile_rows, int32_t* row_of_pair,
                             int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles) {
  SP_REQUIRE(pairs >= 0 && experts > 0 && experts <= 960 && tile_rows > 0, "sp_route_sort: bad sizes");
  SP_REQUIRE(ids && row_of_pair && pair_of_row && tiles && n_tiles, "sp_route_sort: null operand");
  route_sort_kernel<<<1, 1024, 17 * size_t(experts) * sizeof(int32_t), (hipStream_t)stream>>>(
      nullptr, 0, nullptr, 1, const_cast<int32_t*>(ids), pairs, experts, experts, tile_rows, row_of_pair, pair_of_row, tiles,
      n_tiles, RouteRule{0, nullptr, 1, 1, 1.f});
  return check_launch("sp_route_sort");
}

static int route_launch(hipStream_t s, const float* logits, long long stride, int32_t* ids, float* weights, int T, int experts,
                        int tiled, int top, int tile_rows, int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles,
                        int32_t* n_tiles, const RouteRule& rule, const char* what) {
  const size_t lds = 17 * size_t(experts) * sizeof(int32_t);      // first rows, and counts of 16 waves
  if (T <= 256) {      // one block does both: a launch less in the chain of a step of decoded tokens
    route_sort_kernel<<<1, 1024, lds, s>>>(logits, stride, weights, top, ids, T * top, experts, tiled, tile_rows, row_of_pair,
                                           pair_of_row, tiles, n_tiles, rule);
    return check_launch(what);
  }
  const int per_block = experts <= kWaveExperts ? 4 : 256;
  route_topk_kernel<<<(T + per_block - 1) / per_block, 256, 0, s>>>(logits, stride, experts, top, ids, weights, T, rule);
  if (check_launch(what)) return 1;
  route_sort_kernel<<<1, 1024, lds, s>>>(nullptr, 0, nullptr, 1, ids, T * top, experts, tiled, tile_rows, row_of_pair,
                                         pair_of_row, tiles, n_tiles, rule);
  return check_launch(what);
}

extern "C" int sp_route(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top,
                        int tile_rows, int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles) {
  SP_REQUIRE(T >= 0 && experts > 0 && experts <= 960 && top > 0 && top <= experts && tile_rows > 0, "sp_route: bad sizes");
  SP_REQUIRE(logits && ids && weights && row_of_pair && pair_of_row && tiles && n_tiles, "sp_route: null operand");
  return route_launch((hipStream_t)stream, logits, experts, ids, weights, T, experts, experts, top, tile_rows, row_of_pair,
                      pair_of_row, tiles, n_tiles, RouteRule{0, nullptr, 1, 1, 1.f}, "sp_route");
}

extern "C" int sp_route_sigmoid(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top,
                                int tile_rows, int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles) {
  SP_REQUIRE(T >= 0 && experts > 0 && experts <= 960 && top > 0 && top <= experts && tile_rows > 0, "sp_route_sigmoid: bad sizes");
  SP_REQUIRE(logits && ids && weights && row_of_pair && pair_of_row && tiles && n_tiles, "sp_route_sigmoid: null operand");
  return route_launch((hipStream_t)stream, logits, experts, ids, weights, T, experts, experts, top, tile_rows, row_of_pair,
                      pair_of_row, tiles, n_tiles, RouteRule{2, nullptr, 1, 1, 1.f}, "sp_route_sigmoid");
}

extern "C" int sp_route_scored(void* stream, const float* logits, long long stride, const float* correction, int groups,
                               int keep, float scale, int32_t* ids, float* weights, int T, int outputs, int real, int top,
                               int tile_rows, int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles) {
  SP_REQUIRE(T >= 0 && outputs > 0 && outputs <= kWaveExperts && real > 0 && real <= outputs && top > 0 && tile_rows > 0,
             "sp_route_scored: bad sizes (up to %d outputs)", kWaveExperts);
  SP_REQUIRE(groups > 0 && outputs % groups == 0 && keep > 0 && keep <= groups && top <= keep * (outputs / groups),
             "sp_route_scored: %d of %d groups of %d outputs cannot hold %d choices", keep, groups, outputs, top);
  SP_REQUIRE(stride >= outputs, "sp_route_scored: rows of %lld logits for %d outputs", stride, outputs);
  SP_REQUIRE(logits && ids && weights && row_of_pair && pair_of_row && tiles && n_tiles, "sp_route_scored: null operand");
  return route_launch((hipStream_t)stream, logits, stride, ids, weights, T, outputs, real, top, tile_rows, row_of_pair,
                      pair_of_row, tiles, n_tiles, RouteRule{1, correction, groups, keep, scale}, "sp_route_scored");
}

extern "C" int sp_route_combine(void* stream, const float* y, const int32_t* row_of_pair, const float* weights, int top,
                                float* residual, int T, int H) {
  SP_REQUIRE(T >= 0 && H > 0 && top > 0 && y && row_of_pair && residual, "sp_route_combine: bad arguments");
  if (T == 0) return 0;
  route_combine_kernel<float><<<dim3(T, (H + 1023) / 1024), 256, 0, (hipStream_t)stream>>>(y, row_of_pair, weights, top, residual, H,
                                                                                           nullptr, nullptr, 0);
  return check_launch("sp_route_combine");
}

extern "C" int sp_route_combine_identity(void* stream, const float* y, const int32_t* row_of_pair, const float* weights, int top,
                                         const int32_t* ids, int x_dtype, const void* x, int real, float* residual, int T, int H) {
  SP_REQUIRE(T >= 0 && H > 0 && top > 0 && y && row_of_pair && weights && residual && ids && x && real >= 0,
             "sp_route_combine_identity: bad arguments");
  if (T == 0) return 0;
  const dim3 grid(T, (H + 1023) / 1024);
  hipStream_t s = (hipStream_t)stream;
  if (x_dtype == kF32) route_combine_kernel<float><<<grid, 256, 0, s>>>(y, row_of_pair, weights, top, residual, H, ids, (const float*)x, real);
  else if (x_dtype == kBF16) route_combine_kernel<bf16_t><<<grid, 256, 0, s>>>(y, row_of_pair, weights, top, residual, H, ids, (const bf16_t*)x, real);
  else SP_REQUIRE(false, "sp_route_combine_identity: unsupported dtype %d", x_dtype);
  return check_launch("sp_route_combine_identity");
}
