// Grouped products on the matrix cores (bfloat16 operands, float32 sums): the per-head products of attention over
// a latent and the experts of a routed feed-forward, see grouped_gemm.hip for what a group is.
//
// A block of four waves owns a tile of BM rows x BN columns (64 or 128 each) of one group and walks K in steps of
// 64: the rows of a (gathered through the pair list where there is one) and the rows of w go from memory to
// registers to LDS in 16-byte pieces, the next step's pieces asked for before the current step is multiplied.  A
// wave owns a quarter of the tile, as 32x32x16 MFMA tiles.  Rows behind a tile's last row and columns behind N
// are zeros in LDS and are not stored.  Epilogues: store; SiLU(gate) * up with the up rows in a second set of
// accumulators; multiplication by sigmoid of a per-(row, group) gate.
#include "grouped_gemm.h"
#include "mfma.h"
#include "sprout_hip.h"

namespace sprout {

constexpr int GBK = 64;          // step along K
constexpr int GLD = GBK + 8;     // bf16 numbers a row of LDS (16 bytes of padding: neighbouring rows start 4 banks apart)

template <int BM, int BN, int MODE, typename TO>
__global__ __launch_bounds__(256) void grouped_mfma_kernel(GroupedArgs p) {
  constexpr int TM = BM / 64, TN = BN / 64;       // 32x32 tiles of a wave along rows and columns
  constexpr int A_CH = BM / 32, W_CH = BN / 32;   // 16-byte pieces a thread moves per step: rows tid / 8 + 32 j, piece tid % 8
  constexpr bool GATED = MODE == kGated;
  __shared__ __attribute__((aligned(16))) uint16_t As[BM * GLD];
  __shared__ __attribute__((aligned(16))) uint16_t Ws[BN * GLD];
  __shared__ __attribute__((aligned(16))) uint16_t Us[GATED ? BN * GLD : 8];
  int group, row0, nrows;
  if (p.tiles) {
    if (int(blockIdx.x) >= *p.n_tiles) return;
    group = p.tiles[3 * blockIdx.x];
    row0 = p.tiles[3 * blockIdx.x + 1];
    nrows = p.tiles[3 * blockIdx.x + 2];
  } else {
    group = blockIdx.x / p.tiles_per_group;
    row0 = (blockIdx.x - group * p.tiles_per_group) * BM;
    nrows = min(BM, p.rows - row0);
  }
  const int n0 = blockIdx.y * BN;
  const int tid = threadIdx.x, piece = tid & 7, lrow = tid >> 3;
  const uint16_t* a_ptr[A_CH];
  const uint16_t* w_ptr[W_CH];
  const uint16_t* u_ptr[W_CH];
#pragma unroll
  for (int j = 0; j < A_CH; ++j) {
    const int r = lrow + 32 * j;
    a_ptr[j] = nullptr;
    if (r < nrows) {
      const long long src = p.gather ? p.gather[row0 + r] / p.gather_div : row0 + r;
      a_ptr[j] = (const uint16_t*)p.a + src * p.a_stride + group * p.a_group_stride + 8 * piece;
    }
  }
#pragma unroll
  for (int j = 0; j < W_CH; ++j) {
    const int n = n0 + lrow + 32 * j;
    const uint16_t* base = (const uint16_t*)p.w + group * p.w_group_stride + 8 * piece;
    w_ptr[j] = n < p.N ? base + (long long)n * p.K : nullptr;
    u_ptr[j] = (GATED && n < p.N) ? base + (long long)(p.up_offset + n) * p.K : nullptr;
  }
  uint4 a_reg[A_CH], w_reg[W_CH], u_reg[GATED ? W_CH : 1];
  const uint4 zero = make_uint4(0, 0, 0, 0);
  auto fetch = [&](int k0) {
    const bool in_k = k0 + 8 * piece < p.K;      // K is a multiple of 8: a piece is inside or outside as a whole
#pragma unroll
    for (int j = 0; j < A_CH; ++j) a_reg[j] = (a_ptr[j] && in_k) ? ldg128(a_ptr[j] + k0) : zero;
#pragma unroll
    for (int j = 0; j < W_CH; ++j) {
      w_reg[j] = (w_ptr[j] && in_k) ? ldg128(w_ptr[j] + k0) : zero;
      if (GATED) u_reg[j] = (u_ptr[j] && in_k) ? ldg128(u_ptr[j] + k0) : zero;
    }
  };
  const int wave = tid >> 6, lane = tid & 63, lr = lane & 31, lk = lane >> 5;
  const int wm = (wave >> 1) * (BM / 2), wn = (wave & 1) * (BN / 2);
  floatx16 acc[TM][TN], acc2[GATED ? TM : 1][GATED ? TN : 1];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
      if (GATED) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc2[i][j][r] = 0.f;
      }
    }
  fetch(0);
  for (int k0 = 0; k0 < p.K; k0 += GBK) {
#pragma unroll
    for (int j = 0; j < A_CH; ++j) *reinterpret_cast<uint4*>(&As[(lrow + 32 * j) * GLD + 8 * piece]) = a_reg[j];
#pragma unroll
    for (int j = 0; j < W_CH; ++j) {
      *reinterpret_cast<uint4*>(&Ws[(lrow + 32 * j) * GLD + 8 * piece]) = w_reg[j];
      if (GATED) *reinterpret_cast<uint4*>(&Us[(lrow + 32 * j) * GLD + 8 * piece]) = u_reg[j];
    }
    __syncthreads();
    if (k0 + GBK < p.K) fetch(k0 + GBK);
#pragma unroll
    for (int kk = 0; kk < GBK / 16; ++kk) {
      bf16x8 av[TM], wv[TN], uv[GATED ? TN : 1];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        av[i] = as_bf16x8(*reinterpret_cast<const uint4*>(&As[(wm + 32 * i + lr) * GLD + 16 * kk + 8 * lk]));
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        wv[j] = as_bf16x8(*reinterpret_cast<const uint4*>(&Ws[(wn + 32 * j + lr) * GLD + 16 * kk + 8 * lk]));
        if (GATED) uv[j] = as_bf16x8(*reinterpret_cast<const uint4*>(&Us[(wn + 32 * j + lr) * GLD + 16 * kk + 8 * lk]));
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j] = mfma32(av[i], wv[j], acc[i][j]);
          if (GATED) acc2[i][j] = mfma32(av[i], uv[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
  // lane l, number r of a 32x32 tile: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = wm + 32 * i + 8 * (r >> 2) + 4 * lk + (r & 3);
      if (row >= nrows) continue;
      float g = 1.f;
      if (MODE == kSigmoid)
        g = 1.0f / (1.0f + expf(-to_float(((const bf16_t*)p.gate)[(long long)(row0 + row) * p.gate_stride + group])));
      TO* o = (TO*)p.out + (long long)(row0 + row) * p.out_stride + group * p.out_group_stride;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn + 32 * j + lr;
        if (n >= p.N) continue;
        float v = acc[i][j][r];
        if (GATED) v = gated_value(v, acc2[i][j][r], p.act, p.limit);
        if (MODE == kSigmoid) v *= g;
        o[n] = from_float<TO>(v);
      }
    }
}

// Few rows a tile (decoded tokens): tiles of up to 16 rows, a block per tile and 16 columns.  Nothing goes through
// LDS on the way in: a lane takes its 16 bytes of a weight row and of an operand row straight from memory, U = four
// or (long K) eight steps of 32 along K at once (256 or 512 bytes of a row), and the four waves of a block take turns along K, so that a
// product of one row against a whole expert is spread over hundreds of blocks with 64 KB on their way each.  The
// operand rows are the A side of 16x16x32 MFMA tiles; the waves' sums are joined in LDS in a fixed order.
template <int MODE, typename TO, int U>
__global__ __launch_bounds__(256) void grouped_skinny_kernel(GroupedArgs p) {
  constexpr bool GATED = MODE == kGated;
  __shared__ float s_acc[3][64][GATED ? 8 : 4];
  int group, row0, nrows;
  if (p.tiles) {
    if (int(blockIdx.x) >= *p.n_tiles) return;
    group = p.tiles[3 * blockIdx.x];
    row0 = p.tiles[3 * blockIdx.x + 1];
    nrows = p.tiles[3 * blockIdx.x + 2];
  } else {
    group = blockIdx.x / p.tiles_per_group;
    row0 = (blockIdx.x - group * p.tiles_per_group) * 16;
    nrows = min(16, p.rows - row0);
  }
  const int n0 = blockIdx.y * 16;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
  const uint16_t* a_ptr = nullptr;
  if (lr < nrows) {
    const long long src = p.gather ? p.gather[row0 + lr] / p.gather_div : row0 + lr;
    a_ptr = (const uint16_t*)p.a + src * p.a_stride + group * p.a_group_stride + 8 * lj;
  }
  const int n = n0 + lr;
  const uint16_t* base = (const uint16_t*)p.w + group * p.w_group_stride + 8 * lj;
  const uint16_t* w_ptr = n < p.N ? base + (long long)n * p.K : nullptr;
  const uint16_t* u_ptr = (GATED && n < p.N) ? base + (long long)(p.up_offset + n) * p.K : nullptr;
  const uint4 zero = make_uint4(0, 0, 0, 0);
  floatx4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = wave * 32 * U; k0 < p.K; k0 += 4 * 32 * U) {
    uint4 av[U], wv[U], uv[GATED ? U : 1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + 32 * u;
      const bool in_k = k + 8 * lj < p.K;
      wv[u] = (w_ptr && in_k) ? ldg128(w_ptr + k) : zero;
      if (GATED) uv[u] = (u_ptr && in_k) ? ldg128(u_ptr + k) : zero;
      av[u] = (a_ptr && in_k) ? ldg128(a_ptr + k) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc = mfma16(as_bf16x8(av[u]), as_bf16x8(wv[u]), acc);
      if (GATED) acc2 = mfma16(as_bf16x8(av[u]), as_bf16x8(uv[u]), acc2);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s_acc[wave - 1][lane][r] = acc[r];
      if (GATED) s_acc[wave - 1][lane][4 + r] = acc2[r];
    }
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int w = 0; w < 3; ++w)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      acc[r] += s_acc[w][lane][r];
      if (GATED) acc2[r] += s_acc[w][lane][4 + r];
    }
  // lane l, number r: row 4 (l / 16) + r, column l % 16
  if (n >= p.N) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = 4 * lj + r;
    if (row >= nrows) continue;
    float v = acc[r];
    if (GATED) v = gated_value(v, acc2[r], p.act, p.limit);
    if (MODE == kSigmoid)
      v *= 1.0f / (1.0f + expf(-to_float(((const bf16_t*)p.gate)[(long long)(row0 + row) * p.gate_stride + group])));
    ((TO*)p.out)[(long long)(row0 + row) * p.out_stride + group * p.out_group_stride + n] = from_float<TO>(v);
  }
}

bool grouped_mfma_takes(int dtype, const GroupedArgs& p) {
  auto whole = [](long long n) { return n % 8 == 0; };
  return dtype == kBF16 && p.K > 0 && whole(p.K) && whole(p.a_stride) && whole(p.a_group_stride) && whole(p.w_group_stride) &&
         whole((long long)p.up_offset * p.K) && (uintptr_t)p.a % 16 == 0 && (uintptr_t)p.w % 16 == 0;
}

template <int BM, int BN>
static int launch_shape(hipStream_t s, int mode, int out_dtype, const GroupedArgs& p, int tiles, const char* what) {
  dim3 grid(tiles, (p.N + BN - 1) / BN);
  if (mode == kStore && out_dtype == kBF16) grouped_mfma_kernel<BM, BN, kStore, bf16_t><<<grid, 256, 0, s>>>(p);
  else if (mode == kStore && out_dtype == kF32) grouped_mfma_kernel<BM, BN, kStore, float><<<grid, 256, 0, s>>>(p);
  else if (mode == kGated && out_dtype == kBF16) grouped_mfma_kernel<BM, BN, kGated, bf16_t><<<grid, 256, 0, s>>>(p);
  else if (mode == kSigmoid && out_dtype == kBF16) grouped_mfma_kernel<BM, BN, kSigmoid, bf16_t><<<grid, 256, 0, s>>>(p);
  else SP_REQUIRE(false, "%s: no matrix-core kernel for epilogue %d with output type %d", what, mode, out_dtype);
  return check_launch(what);
}

template <int U>
static int launch_skinny_u(hipStream_t s, int mode, int out_dtype, const GroupedArgs& p, int tiles, const char* what) {
  dim3 grid(tiles, (p.N + 15) / 16);
  if (mode == kStore && out_dtype == kBF16) grouped_skinny_kernel<kStore, bf16_t, U><<<grid, 256, 0, s>>>(p);
  else if (mode == kStore && out_dtype == kF32) grouped_skinny_kernel<kStore, float, U><<<grid, 256, 0, s>>>(p);
  else if (mode == kGated && out_dtype == kBF16) grouped_skinny_kernel<kGated, bf16_t, U><<<grid, 256, 0, s>>>(p);
  else if (mode == kSigmoid && out_dtype == kBF16) grouped_skinny_kernel<kSigmoid, bf16_t, U><<<grid, 256, 0, s>>>(p);
  else SP_REQUIRE(false, "%s: no matrix-core kernel for epilogue %d with output type %d", what, mode, out_dtype);
  return check_launch(what);
}

static int launch_skinny(hipStream_t s, int mode, int out_dtype, const GroupedArgs& p, int tiles, const char* what) {
  // a wave's turn along K is 32 U numbers: eight steps at once where K gives every wave two turns of them
  return p.K >= 2048 ? launch_skinny_u<8>(s, mode, out_dtype, p, tiles, what) : launch_skinny_u<4>(s, mode, out_dtype, p, tiles, what);
}

int launch_grouped_mfma(hipStream_t s, int mode, int out_dtype, const GroupedArgs& p, int tiles, int tile_rows,
                        const char* what) {
  SP_REQUIRE(tile_rows == 16 || tile_rows == 64 || tile_rows == 128 || tile_rows == 256, "%s: tiles of %d rows", what, tile_rows);
  if (tile_rows == 16) return launch_skinny(s, mode, out_dtype, p, tiles, what);
  // wide tiles where there are columns for them; the gated epilogue keeps two sets of accumulators, so its tiles of
  // 256 rows are narrow.  Tiles of 256 rows hold a group's rows in one block where they can: its weights are then
  // fetched once, not once per tile.
  const bool wide = p.N > 64;
  if (tile_rows == 256) return (wide && mode != kGated) ? launch_shape<256, 128>(s, mode, out_dtype, p, tiles, what)
                                                        : launch_shape<256, 64>(s, mode, out_dtype, p, tiles, what);
  if (tile_rows == 128) return wide ? launch_shape<128, 128>(s, mode, out_dtype, p, tiles, what)
                                    : launch_shape<128, 64>(s, mode, out_dtype, p, tiles, what);
  return wide ? launch_shape<64, 128>(s, mode, out_dtype, p, tiles, what)
              : launch_shape<64, 64>(s, mode, out_dtype, p, tiles, what);
}

}  // namespace sprout
