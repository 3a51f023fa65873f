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
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float best_z = 0.f;
    for (int e = 0; e < experts; ++e) {
      const float v = z[e];
      bool taken = false;
      for (int j = 0; j < k; ++j) taken |= id[j] == e;
      if (!taken && (best < 0 || v > best_z)) { best = e; best_z = v; }
    }
    id[k] = best;
    w[k] = best_z;
  }
  const float top_z = w[0];
  float sum = 0.f;
  for (int k = 0; k < top; ++k) { w[k] = expf(w[k] - top_z); sum += w[k]; }
  for (int k = 0; k < top; ++k) w[k] /= sum;
}

// One thread a token.
__global__ void route_topk_kernel(const float* __restrict__ logits, int experts, int top, int32_t* __restrict__ ids,
                                  float* __restrict__ weights, int T) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  route_token(logits + size_t(t) * experts, experts, top, ids + size_t(t) * top, weights + size_t(t) * top);
}

// One block: sorts the pairs (token, choice) by expert.  row_of_pair[p] = the row of pair p in the sorted order,
// pair_of_row its inverse; tiles [n][3] = (expert, first row, rows) cuts every expert's rows into tiles of at most
// tile_rows; *n_tiles = n.  Within an expert the rows stand in no fixed order (every row is computed for itself).
// With `logits` (and `weights`, `top`) the block first makes the choice itself (ids and weights are then outputs):
// choice and order in one launch.
__global__ void route_sort_kernel(const float* __restrict__ logits, float* __restrict__ weights, int top,
                                  int32_t* __restrict__ ids, int pairs, int experts, int tile_rows,
                                  int32_t* __restrict__ row_of_pair, int32_t* __restrict__ pair_of_row,
                                  int32_t* __restrict__ tiles, int32_t* __restrict__ n_tiles) {
  extern __shared__ int32_t count[];      // [experts] counts, then [experts] first rows
  int32_t* first = count + experts;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
  if (logits)
    for (int t = threadIdx.x; t < pairs / top; t += blockDim.x)
      route_token(logits + size_t(t) * experts, experts, top, ids + size_t(t) * top, weights + size_t(t) * top);
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) row_of_pair[p] = atomicAdd(&count[ids[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int row = 0, n = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = row;
      for (int r = 0; r < count[e]; r += tile_rows) {
        tiles[3 * n] = e;
        tiles[3 * n + 1] = row + r;
        tiles[3 * n + 2] = min(tile_rows, count[e] - r);
        ++n;
      }
      row += count[e];
    }
    *n_tiles = n;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int row = first[ids[p]] + row_of_pair[p];
    row_of_pair[p] = row;
    pair_of_row[row] = p;
  }
}

// residual[t] += sum over the token's choices, in their order, of weight * (the expert's output row).
__global__ void route_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ row_of_pair,
                                     const float* __restrict__ weights, int top, float* __restrict__ residual, int H) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float sum = 0.f;
    for (int k = 0; k < top; ++k)
      sum = fmaf(weights[size_t(t) * top + k], y[size_t(row_of_pair[size_t(t) * top + k]) * H + i], sum);
    residual[size_t(t) * H + i] += sum;
  }
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_route_topk(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top) {
  SP_REQUIRE(T >= 0 && experts > 0 && top > 0 && top <= experts, "sp_route_topk: %d of %d experts", top, experts);
  SP_REQUIRE(logits && ids && weights, "sp_route_topk: null operand");
  if (T == 0) return 0;
  route_topk_kernel<<<(T + 63) / 64, 64, 0, (hipStream_t)stream>>>(logits, experts, top, ids, weights, T);
  return check_launch("sp_route_topk");
}

extern "C" int sp_route_max_tiles(int pairs, int experts, int tile_rows) {
  // every expert's last tile may be a partial one
  return (pairs + tile_rows - 1) / tile_rows + (pairs < experts ? pairs : experts);
}

extern "C" int sp_route_sort(void* stream, const int32_t* ids, int pairs, int experts, int tile_rows, int32_t* row_of_pair,
                             int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles) {
  SP_REQUIRE(pairs >= 0 && experts > 0 && experts <= 8192 && tile_rows > 0, "sp_route_sort: bad sizes");
  SP_REQUIRE(ids && row_of_pair && pair_of_row && tiles && n_tiles, "sp_route_sort: null operand");
  route_sort_kernel<<<1, 1024, 2 * size_t(experts) * sizeof(int32_t), (hipStream_t)stream>>>(
      nullptr, nullptr, 1, const_cast<int32_t*>(ids), pairs, experts, tile_rows, row_of_pair, pair_of_row, tiles, n_tiles);
  return check_launch("sp_route_sort");
}

extern "C" int sp_route(void* stream, const float* logits, int32_t* ids, float* weights, int T, int experts, int top,
                        int tile_rows, int32_t* row_of_pair, int32_t* pair_of_row, int32_t* tiles, int32_t* n_tiles) {
  SP_REQUIRE(T >= 0 && experts > 0 && experts <= 8192 && top > 0 && top <= experts && tile_rows > 0, "sp_route: bad sizes");
  SP_REQUIRE(logits && ids && weights && row_of_pair && pair_of_row && tiles && n_tiles, "sp_route: null operand");
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = 2 * size_t(experts) * sizeof(int32_t);
  if (T <= 8192) {      // one block does both: a launch less in the chain of a step
    route_sort_kernel<<<1, 1024, lds, s>>>(logits, weights, top, ids, T * top, experts, tile_rows, row_of_pair, pair_of_row,
                                           tiles, n_tiles);
    return check_launch("sp_route");
  }
  route_topk_kernel<<<(T + 63) / 64, 64, 0, s>>>(logits, experts, top, ids, weights, T);
  if (check_launch("sp_route (choice)")) return 1;
  route_sort_kernel<<<1, 1024, lds, s>>>(nullptr, nullptr, 1, ids, T * top, experts, tile_rows, row_of_pair, pair_of_row,
                                         tiles, n_tiles);
  return check_launch("sp_route (order)");
}

extern "C" int sp_route_combine(void* stream, const float* y, const int32_t* row_of_pair, const float* weights, int top,
                                float* residual, int T, int H) {
  SP_REQUIRE(T >= 0 && H > 0 && top > 0 && y && row_of_pair && weights && residual, "sp_route_combine: bad arguments");
  if (T == 0) return 0;
  route_combine_kernel<<<T, 256, 0, (hipStream_t)stream>>>(y, row_of_pair, weights, top, residual, H);
  return check_launch("sp_route_combine");
}
