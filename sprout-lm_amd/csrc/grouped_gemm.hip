// Products of many small groups in one launch: a group (an attention head, an expert) has weights [N, K] of its
// own and multiplies its own rows.  One kernel serves the per-head products of attention over a latent (every
// group owns all tokens, its operand a column range of the row) and the experts of a routed feed-forward (a
// group owns the rows that were routed to it, listed in tiles that a kernel built on the device).
//
// This file holds the float32-arithmetic form (FMA, any sizes and both storage types): tiles of 64 rows x 64
// columns, steps of 16 along K through LDS, a thread a 4 x 4 patch.
#include "grouped_gemm.h"
#include "sprout_hip.h"

namespace sprout {

constexpr int GT = 64;     // rows and columns of a tile
constexpr int GK = 16;     // step along K

template <typename TA, typename TO, int MODE>
__global__ __launch_bounds__(256) void grouped_kernel(GroupedArgs p) {
  int group, row0, nrows;
  if (p.tiles) {
    if (int(blockIdx.x) >= *p.n_tiles) return;
    group = p.tiles[3 * blockIdx.x];
    row0 = p.tiles[3 * blockIdx.x + 1];
    nrows = p.tiles[3 * blockIdx.x + 2];
  } else {
    group = blockIdx.x / p.tiles_per_group;
    row0 = (blockIdx.x - group * p.tiles_per_group) * GT;
    nrows = min(GT, p.rows - row0);
  }
  const int n0 = blockIdx.y * GT;
  __shared__ float As[GK][GT + 4];
  __shared__ float Ws[GK][GT + 4];
  __shared__ float Us[MODE == kGated ? GK : 1][GT + 4];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int lk = tid & 15, lr = tid >> 4;      // this thread loads column lk of rows lr, lr + 16, lr + 32, lr + 48
  const TA* a_rows[4];
  const TA* w_rows[4];
  const TA* u_rows[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = lr + 16 * j;
    a_rows[j] = nullptr;
    if (r < nrows) {
      const long long src = p.gather ? p.gather[row0 + r] / p.gather_div : row0 + r;
      a_rows[j] = (const TA*)p.a + src * p.a_stride + group * p.a_group_stride;
    }
    const int n = n0 + r;
    w_rows[j] = n < p.N ? (const TA*)p.w + group * p.w_group_stride + (long long)n * p.K : nullptr;
    u_rows[j] = (MODE == kGated && n < p.N) ? (const TA*)p.w + group * p.w_group_stride + (long long)(p.up_offset + n) * p.K : nullptr;
  }
  float acc[4][4] = {}, acc2[4][4] = {};
  for (int k0 = 0; k0 < p.K; k0 += GK) {
    const bool in_k = k0 + lk < p.K;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      As[lk][lr + 16 * j] = (a_rows[j] && in_k) ? to_float(a_rows[j][k0 + lk]) : 0.f;
      Ws[lk][lr + 16 * j] = (w_rows[j] && in_k) ? to_float(w_rows[j][k0 + lk]) : 0.f;
      if (MODE == kGated) Us[lk][lr + 16 * j] = (u_rows[j] && in_k) ? to_float(u_rows[j][k0 + lk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      float av[4], wv[4], uv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = As[k][ty * 4 + i];
        wv[i] = Ws[k][tx * 4 + i];
        if (MODE == kGated) uv[i] = Us[k][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
          if (MODE == kGated) acc2[i][j] = fmaf(av[i], uv[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= nrows) continue;
    float g = 1.f;
    if (MODE == kSigmoid) g = 1.0f / (1.0f + expf(-to_float(((const TA*)p.gate)[(long long)(row0 + r) * p.gate_stride + group])));
    TO* o = (TO*)p.out + (long long)(row0 + r) * p.out_stride + group * p.out_group_stride;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      float v = acc[i][j];
      if (MODE == kGated) v = gated_value(v, acc2[i][j], p.act, p.limit);
      if (MODE == kSigmoid) v *= g;
      o[n] = from_float<TO>(v);
    }
  }
}

template <int MODE>
static int launch_grouped(hipStream_t s, int dtype, int out_dtype, const GroupedArgs& p, int blocks_x, const char* what) {
  dim3 grid(blocks_x, (p.N + GT - 1) / GT);
  if (dtype == kF32 && out_dtype == kF32) grouped_kernel<float, float, MODE><<<grid, 256, 0, s>>>(p);
  else if (dtype == kBF16 && out_dtype == kBF16) grouped_kernel<bf16_t, bf16_t, MODE><<<grid, 256, 0, s>>>(p);
  else if (dtype == kBF16 && out_dtype == kF32) grouped_kernel<bf16_t, float, MODE><<<grid, 256, 0, s>>>(p);
  else SP_REQUIRE(false, "%s: unsupported dtypes %d -> %d", what, dtype, out_dtype);
  return check_launch(what);
}

}  // namespace sprout

using namespace sprout;

// Rows a tile of the grouped products holds.  Where the matrix-core kernels take the operands (bfloat16, K in
// eights): 16 where a group has at most 8 rows on average (decoded tokens), 256 from 192 on, 128 from 96 on (measured at 256
// rows a group: tiles of 256, half empty every other time, still beat tiles of 128: 87 against 103 us); 64 in
// between and for every other operand.
extern "C" int sp_group_tile_rows(int dtype, long long rows, int groups, int K) {
  if (dtype != kBF16 || K % 8 || groups <= 0) return GT;
  const long long each = rows / groups;
  if (rows <= 8ll * groups) return 16;
  return each >= 192 ? 256 : each >= 96 ? 128 : GT;
}

// The float32-arithmetic kernel cuts its own tiles of 64 rows; a list cut for more rows is not for it.
static int grouped(hipStream_t s, int mode, int dtype, int out_dtype, const GroupedArgs& p, int tiles, int tile_rows,
                   const char* what) {
  if (grouped_mfma_takes(dtype, p)) {
    // many rows a group, from a tile list: the pipelined tiled kernel (its two epilogues are the experts')
    if (p.tiles && tile_rows >= 128 && p.K % 64 == 0 && p.a_group_stride == 0 && p.a_stride == p.K &&
        ((mode == kGated && out_dtype == kBF16 && p.up_offset == p.N && p.out_stride == p.N) ||
         (mode == kStore && out_dtype == kF32 && p.out_stride == p.N)) && p.out_group_stride == 0)
      return grouped_pipe(s, mode == kGated, p.act, p.limit, p.a, p.w, p.w_group_stride, p.tiles, p.n_tiles, tiles, tile_rows, p.gather,
                          p.gather_div, p.out, p.N, p.K, what);
    return launch_grouped_mfma(s, mode, out_dtype, p, tiles, tile_rows, what);
  }
  SP_REQUIRE(tile_rows == GT, "%s: tiles of %d rows need operands the matrix-core kernels take", what, tile_rows);
  if (mode == kGated) return launch_grouped<kGated>(s, dtype, out_dtype, p, tiles, what);
  if (mode == kSigmoid) return launch_grouped<kSigmoid>(s, dtype, out_dtype, p, tiles, what);
  return launch_grouped<kStore>(s, dtype, out_dtype, p, tiles, what);
}

extern "C" int sp_head_gemm(void* stream, int dtype, const void* a, long long a_stride, long long a_head_stride,
                            const void* w, void* out, long long out_stride, long long out_head_stride, const void* gate,
                            long long gate_stride, int T, int heads, int N, int K) {
  SP_REQUIRE(T >= 0 && heads > 0 && N > 0 && K > 0, "sp_head_gemm: bad sizes T=%d heads=%d N=%d K=%d", T, heads, N, K);
  SP_REQUIRE(a && w && out, "sp_head_gemm: null operand");
  SP_REQUIRE(a_stride >= (heads - 1) * a_head_stride + K && out_stride >= (heads - 1) * out_head_stride + N &&
                 (!gate || gate_stride >= heads), "sp_head_gemm: a row does not hold every head's numbers");
  if (T == 0) return 0;
  GroupedArgs p = {};
  p.a = a; p.a_stride = a_stride; p.a_group_stride = a_head_stride;
  p.w = w; p.w_group_stride = (long long)N * K;
  p.out = out; p.out_stride = out_stride; p.out_group_stride = out_head_stride;
  p.gate = gate; p.gate_stride = gate_stride;
  p.rows = T;
  p.N = N; p.K = K;
  const int tile_rows = !grouped_mfma_takes(dtype, p) ? GT : T <= 32 ? 16 : T >= 256 ? 128 : GT;
  p.tiles_per_group = (T + tile_rows - 1) / tile_rows;
  const long long blocks = (long long)heads * p.tiles_per_group;
  SP_REQUIRE(blocks < (1ll << 31), "sp_head_gemm: too many tiles");
  return grouped((hipStream_t)stream, gate ? kSigmoid : kStore, dtype, dtype, p, int(blocks), tile_rows, "sp_head_gemm");
}

extern "C" int sp_expert_gate_up(void* stream, int dtype, const void* x, const void* w, const int32_t* tiles,
                                 const int32_t* n_tiles, int max_tiles, int tile_rows, const int32_t* pair_of_row, int top,
                                 void* out, int T, int experts, int inner, int K, int activation, float limit) {
  SP_REQUIRE(activation >= 0 && activation < kGateActs, "sp_expert_gate_up: no kernel for activation %d", activation);
  SP_REQUIRE(T >= 0 && experts > 0 && inner > 0 && K > 0 && top > 0 && max_tiles > 0, "sp_expert_gate_up: bad sizes");
  SP_REQUIRE(x && w && tiles && n_tiles && pair_of_row && out, "sp_expert_gate_up: null operand");
  if (T == 0) return 0;
  GroupedArgs p = {};
  p.a = x; p.a_stride = K; p.gather = pair_of_row; p.gather_div = top;
  p.w = w; p.w_group_stride = 2ll * inner * K;
  p.out = out; p.out_stride = inner;
  p.tiles = tiles; p.n_tiles = n_tiles;
  p.N = inner; p.K = K; p.up_offset = inner;
  p.act = activation; p.limit = limit;
  return grouped((hipStream_t)stream, kGated, dtype, dtype, p, max_tiles, tile_rows, "sp_expert_gate_up");
}

extern "C" int sp_expert_down(void* stream, int dtype, const void* act, const void* w, const int32_t* tiles,
                              const int32_t* n_tiles, int max_tiles, int tile_rows, float* out, int rows, int experts,
                              int hidden, int inner) {
  SP_REQUIRE(rows >= 0 && experts > 0 && inner > 0 && hidden > 0 && max_tiles > 0, "sp_expert_down: bad sizes");
  SP_REQUIRE(act && w && tiles && n_tiles && out, "sp_expert_down: null operand");
  if (rows == 0) return 0;
  GroupedArgs p = {};
  p.a = act; p.a_stride = inner;
  p.w = w; p.w_group_stride = (long long)hidden * inner;
  p.out = out; p.out_stride = hidden;
  p.tiles = tiles; p.n_tiles = n_tiles;
  p.N = hidden; p.K = inner;
  return grouped((hipStream_t)stream, kStore, dtype, kF32, p, max_tiles, tile_rows, "sp_expert_down");
}
