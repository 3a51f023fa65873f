// Routing of a feed-forward with experts: choice of the experts, the order in which the grouped products walk
// the (token, choice) pairs, and the weighted sum of the experts' outputs.  Everything float32; nothing is
// decided on the host, so a step can be recorded into a graph.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

// The `top` largest of a token's `experts` logits (the lowest index wins a tie), in falling order, and the softmax
// over the chosen logits alone.
__device__ __forceinline__ void route_token(const float* __restrict__ z, int experts, int top, int32_t* __restrict__ id,
                                            float* __restrict__ w) {
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
    const float ex = expf(best_z - top_z);
    sum += ex;
    id[k] = best;
    w[k] = ex;
    prev = best;
    prev_z = best_z;
  }
  const float scale = 1.0f / sum;
  for (int k = 0; k < top; ++k) w[k] *= scale;
}

// The same choice by a whole wave, for up to 256 experts: lane l holds the logits of experts l, l + 64, ..., one
// coalesced load, and every choice is a reduction over the wave (larger value first, lower index among equals).
constexpr int kWaveExperts = 256;
__device__ __forceinline__ void route_token_wave(const float* __restrict__ z, int experts, int top, int32_t* __restrict__ id,
                                                 float* __restrict__ w, int lane) {
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
    const float ex = expf(bv - top_z);
    sum += ex;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (k == lane + 64 * j) { my_id[j] = be; my_ex[j] = ex; }
  }
  const float scale = 1.0f / sum;
#pragma unroll
  for (int j = 0; j < J; ++j)
    if (lane + 64 * j < top) { id[lane + 64 * j] = my_id[j]; w[lane + 64 * j] = my_ex[j] * scale; }
}

// A wave a token (up to 256 experts), else a thread a token.
__global__ void route_topk_kernel(const float* __restrict__ logits, int experts, int top, int32_t* __restrict__ ids,
                                  float* __restrict__ weights, int T) {
  if (experts <= kWaveExperts) {
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t < T) route_token_wave(logits + size_t(t) * experts, experts, top, ids + size_t(t) * top, weights + size_t(t) * top, threadIdx.x & 63);
    return;
  }
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  route_token(logits + size_t(t) * experts, experts, top, ids + size_t(t) * top, weights + size_t(t) * top);
}

// One block: sorts the pairs (token, choice) by expert.  row_of_pair[p] = the row of pair p in the sorted order,
// pair_of_row its inverse; tiles [n][3] = (expert, first row, rows) cuts every expert's rows into tiles of at most
// tile_rows; *n_tiles = n.  Within an expert the rows of a wave's run of pairs stand together, in no
// fixed order (every row is computed for itself).  A wave owns a run of pairs and counts them in a row of LDS
// counters of its own (counts [waves][experts]), so an atomic meets at most the 63 other lanes of its instruction.
// With `logits` (and `weights`, `top`) the block first makes the choice itself (ids and weights are then outputs):
// choice and order in one launch.
__global__ __launch_bounds__(1024) void route_sort_kernel(const float* __restrict__ logits, float* __restrict__ weights,
                                                          int top, int32_t* __restrict__ ids, int pairs, int experts,
                                                          int tile_rows, int32_t* __restrict__ row_of_pair,
                                                          int32_t* __restrict__ pair_of_row, int32_t* __restrict__ tiles,
                                                          int32_t* __restrict__ n_tiles) {
  extern __shared__ int32_t lds[];      // [experts] first rows, then [waves][experts] counts
  const int waves = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int32_t* first = lds;
  int32_t* mine = lds + experts + wave * experts;
  for (int i = threadIdx.x; i < waves * experts; i += blockDim.x) lds[experts + i] = 0;
  if (logits) {
    if (experts <= kWaveExperts)
      for (int t = wave; t < pairs / top; t += waves)
        route_token_wave(logits + size_t(t) * experts, experts, top, ids + size_t(t) * top, weights + size_t(t) * top, lane);
    else
      for (int t = threadIdx.x; t < pairs / top; t += blockDim.x)
        route_token(logits + size_t(t) * experts, experts, top, ids + size_t(t) * top, weights + size_t(t) * top);
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
      for (int r = 0; r < count; r += tile_rows) {
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
// token and 1,024 columns, a thread four neighbouring columns where rows are in fours.
__global__ __launch_bounds__(256) void route_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ row_of_pair,
                                                            const float* __restrict__ weights, int top,
                                                            float* __restrict__ residual, int H) {
  const int t = blockIdx.x;
  const int32_t* rows = row_of_pair + size_t(t) * top;
  const float* wt = weights + size_t(t) * top;
  if ((H & 3) == 0) {
    const int i = 4 * (blockIdx.y * 256 + threadIdx.x);
    if (i >= H) return;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < top; ++k) {
      const float w = wt[k];
      const float4 v = *reinterpret_cast<const float4*>(y + size_t(rows[k]) * H + i);
      sum.x = fmaf(w, v.x, sum.x); sum.y = fmaf(w, v.y, sum.y); sum.z = fmaf(w, v.z, sum.z); sum.w = fmaf(w, v.w, sum.w);
    }
    float4* r = reinterpret_cast<float4*>(residual + size_t(t) * H + i);
    const float4 old = *r;
    *r = make_float4(old.x + sum.x, old.y + sum.y, old.z + sum.z, old.w + sum.w);
    return;
  }
  for (int i = blockIdx.y * 1024 + threadIdx.x; i < min(H, (int(blockIdx.y) + 1) * 1024); i += 256) {
    float sum = 0.f;
    for (int k = 0; k < top; ++k) sum = fmaf(wt[k], y[size_t(rows[k]) * H + i], sum);
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
  route_topk_kernel<<<(T + per_block - 1) / per_block, 256, 0, (hipStream_t)stream>>>(logits, experts, top, ids, weights, T);
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
      nullptr, nullptr, 1, const_cast<int32_t*>(ids), pairs, experts, tile_rows, row_of_pair, pair_of_row, tiles, n_tiles);
  return check_launch("sp_route_sort");
}

extern "C" int sp_route(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top,
                        int tile_rows, int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles) {
  SP_REQUIRE(T >= 0 && experts > 0 && experts <= 960 && top > 0 && top <= experts && tile_rows > 0, "sp_route: bad sizes");
  SP_REQUIRE(logits && ids && weights && row_of_pair && pair_of_row && tiles && n_tiles, "sp_route: null operand");
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = 17 * size_t(experts) * sizeof(int32_t);      // first rows, and counts of 16 waves
  if (T <= 256) {      // one block does both: a launch less in the chain of a step of decoded tokens
    route_sort_kernel<<<1, 1024, lds, s>>>(logits, weights, top, ids, T * top, experts, tile_rows, row_of_pair, pair_of_row,
                                           tiles, n_tiles);
    return check_launch("sp_route");
  }
  const int per_block = experts <= kWaveExperts ? 4 : 256;
  route_topk_kernel<<<(T + per_block - 1) / per_block, 256, 0, s>>>(logits, experts, top, ids, weights, T);
  if (check_launch("sp_route (choice)")) return 1;
  route_sort_kernel<<<1, 1024, lds, s>>>(nullptr, nullptr, 1, ids, T * top, experts, tile_rows, row_of_pair, pair_of_row,
                                         tiles, n_tiles);
  return check_launch("sp_route (order)");
}

extern "C" int sp_route_combine(void* stream, const float* y, const int32_t* row_of_pair, const float* weights, int top,
                                float* residual, int T, int H) {
  SP_REQUIRE(T >= 0 && H > 0 && top > 0 && y && row_of_pair && weights && residual, "sp_route_combine: bad arguments");
  if (T == 0) return 0;
  route_combine_kernel<<<dim3(T, (H + 1023) / 1024), 256, 0, (hipStream_t)stream>>>(y, row_of_pair, weights, top, residual, H);
  return check_launch("sp_route_combine");
}
