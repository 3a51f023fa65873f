// The experts' products for many rows (prompts) on the pipelined tiled kernel of gemm_pipe.h in its grouped form:
// tiles of 256 or 128 rows of one expert each, operand rows gathered through the pair list straight into LDS, the
// expert's weights behind a stride.  Epilogues: act(gate, up) (the weights hold an expert's gate rows, then its up
// rows) into bfloat16, or a float32 store.
#include "gemm_pipe.h"

namespace sprout {

int grouped_pipe(hipStream_t s, bool gated, int act, float limit, const void* x, const void* w, long long w_group_stride, const int32_t* tiles,
                 const int32_t* n_tiles, int max_tiles, int tile_rows, const int32_t* gather, int gather_div, void* out,
                 int N, int K, const char* what) {
  SP_REQUIRE(K > 0 && K % 64 == 0 && (tile_rows == 128 || tile_rows == 256), "%s: K=%d, tiles of %d rows", what, K, tile_rows);
  const PipeGroups groups = {tiles, n_tiles, gather, gather_div > 0 ? gather_div : 1, w_group_stride};
  const uint16_t *xp = (const uint16_t*)x, *wp = (const uint16_t*)w;
  RopeArgs epilogue = {};
  epilogue.act = act;
  epilogue.limit = limit;
  if (tile_rows == 256)
    return gated ? launch_pipe_grouped<2, 2, 4, 2, 3, kSilu>(s, xp, wp, out, N, K, max_tiles, groups, what, epilogue)
                 : launch_pipe_grouped<2, 2, 4, 2, 3, kStoreF32>(s, xp, wp, out, N, K, max_tiles, groups, what);
  return gated ? launch_pipe_grouped<1, 2, 4, 2, 4, kSilu>(s, xp, wp, out, N, K, max_tiles, groups, what, epilogue)
               : launch_pipe_grouped<1, 2, 4, 2, 4, kStoreF32>(s, xp, wp, out, N, K, max_tiles, groups, what);
}

}  // namespace sprout
