// Arguments shared by the grouped product kernels (float32 arithmetic in grouped_gemm.hip, matrix cores in
// grouped_gemm_bf16.hip).
#pragma once
#include "common.h"

namespace sprout {

struct GroupedArgs {
  const void* a;            // operand rows
  long long a_stride;       // between rows
  long long a_group_stride; // between the groups' column ranges of a row (0: every group reads the same columns)
  const int32_t* gather;    // row r of the list reads operand row gather[r] / gather_div (null: row r)
  int gather_div;
  const void* w;            // [groups][rows of K]
  long long w_group_stride;
  void* out;
  long long out_stride, out_group_stride;
  const void* gate;         // epilogue 2: out *= sigmoid(gate[row * gate_stride + group])
  long long gate_stride;
  const int32_t* tiles;     // [n][3] = group, first row, rows (null: every group owns `rows`, in tiles_per_group tiles)
  const int32_t* n_tiles;
  int rows, tiles_per_group;
  int N, K;
  int up_offset;            // epilogue 1: weight row n is the gate's, row up_offset + n the matching up row
  int act;                  // epilogue 1: which gated activation (GateAct), and its limit
  float limit;
};

enum { kStore = 0, kGated = 1, kSigmoid = 2 };

// Whether the matrix-core kernels take these operands: bfloat16, K in whole groups of 8, and every row of a and w
// starting at a multiple of 16 bytes.
bool grouped_mfma_takes(int dtype, const GroupedArgs& p);
// tile_rows: 16, 64, 128 or 256 rows a tile (with a tile list: the size the list was cut for).
int launch_grouped_mfma(hipStream_t s, int mode, int out_dtype, const GroupedArgs& p, int tiles, int tile_rows,
                        const char* what);

// The pipelined tiled kernel in its grouped form (grouped_gemm_pipe.hip): tiles of 128 or 256 rows from a tile list,
// K in whole steps of 64, bfloat16; `gated`: act(gate, up) into bfloat16, else a float32 store.
int grouped_pipe(hipStream_t s, bool gated, int act, float limit, const void* x, const void* w, long long w_group_stride, const int32_t* tiles,
                 const int32_t* n_tiles, int max_tiles, int tile_rows, const int32_t* gather, int gather_div, void* out,
                 int N, int K, const char* what);

}  // namespace sprout
