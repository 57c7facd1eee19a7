// Launchers of the GEMM kernel instantiations.  Each workgroup tile is compiled in its own
// translation unit (gemm_tiles.hip, once per tile) so that the build runs them in parallel.
#pragma once
#include <hip/hip_runtime.h>

#include "gemm_mfma.hpp"

namespace tenmo {

// One workgroup per tile (grid.y = K slices).  false: no variant for these operand modes.
// (bsum: also add up the column sums of B, see BsumArgs — both operands with unit stride along M / N only, false otherwise;
// the same argument of the stream-K launchers below)
bool launch_gemm_256x128(const GemmArgs& g, dim3 grid, int amode, int bmode, hipStream_t stream, const BsumArgs* bsum = nullptr);
bool launch_gemm_128x128(const GemmArgs& g, dim3 grid, int amode, int bmode, hipStream_t stream, const BsumArgs* bsum = nullptr);
bool launch_gemm_64x64(const GemmArgs& g, dim3 grid, int amode, int bmode, hipStream_t stream, const BsumArgs* bsum = nullptr);
bool launch_gemm_128x64(const GemmArgs& g, dim3 grid, int amode, int bmode, hipStream_t stream, const BsumArgs* bsum = nullptr);
bool launch_gemm_64x128(const GemmArgs& g, dim3 grid, int amode, int bmode, hipStream_t stream, const BsumArgs* bsum = nullptr);

// Two products with the 64x64 tile in one launch (count0 / count1 workgroups).  false: no variant for these operand modes.
bool launch_gemm_pair_64x64(const GemmArgs& g0, const GemmArgs& g1, unsigned count0, unsigned count1, int amode0, int bmode0, int amode1, int bmode1,
                            hipStream_t stream);

// C[kept batch] (+)= the sum over the reduced batch dimensions `red` of A . B (gemm_reduce_kernel): `wgs` = kept batches x
// tiles of the chosen size (g.tiles_m, g.tiles_n set for it; g.batch, g.batch_count = the kept dimensions).  Vector
// operand modes only; false: no variant for these modes.
bool launch_gemm_reduce_128x128(const GemmArgs& g, const BatchReduce& red, unsigned wgs, int amode, int bmode, hipStream_t stream);
bool launch_gemm_reduce_64x64(const GemmArgs& g, const BatchReduce& red, unsigned wgs, int amode, int bmode, hipStream_t stream);

// Stream-K: `wgs` persistent workgroups, then the fix-up over `tiles` tiles in `fix_parts` parts
// each (0: no tile is shared, no fix-up).  Vector operand modes only.
bool launch_streamk_256x128(const GemmArgs& g, const StreamKArgs& sk, unsigned wgs, unsigned tiles, unsigned fix_parts, int amode, int bmode, hipStream_t stream,
                            const BsumArgs* bsum = nullptr);
bool launch_streamk_128x128(const GemmArgs& g, const StreamKArgs& sk, unsigned wgs, unsigned tiles, unsigned fix_parts, int amode, int bmode, hipStream_t stream,
                            const BsumArgs* bsum = nullptr);
bool launch_streamk_128x64(const GemmArgs& g, const StreamKArgs& sk, unsigned wgs, unsigned tiles, unsigned fix_parts, int amode, int bmode, hipStream_t stream,
                            const BsumArgs* bsum = nullptr);
bool launch_streamk_64x64(const GemmArgs& g, const StreamKArgs& sk, unsigned wgs, unsigned tiles, unsigned fix_parts, int amode, int bmode, hipStream_t stream,
                            const BsumArgs* bsum = nullptr);

// Short reduction (K up to 64), vector operand modes, plain or accumulating store: persistent workgroups that hold a
// whole tile's operands in LDS, loaded one tile ahead by wavefronts of their own (gemm_smallk.hip).  `total_tiles` =
// batches x 64x64 tiles (g.tiles_m, g.tiles_n set for that tile).  The caller has checked what the direct loads need
// (pitches, an MN-major extent divisible by 4, K % 4 == 0 for a K-major operand when K is no multiple of 16).
// `by_batch`: order the tiles for the XCDs (whole batches, or whole column blocks).  false: not a shape this kernel takes.
bool launch_gemm_smallk_64x64(const GemmArgs& g, int amode, int bmode, unsigned cus, unsigned total_tiles, bool by_batch, hipStream_t stream);

// Persistent workgroups that treat the K steps of all their tiles as one stream through a deep LDS ring, with wavefronts
// of their own for the loads, two such workgroups per CU (gemm_panel.hip): for a
// short or medium reduction into a result of many tiles.  Vector operand modes, plain or accumulating store.
// `total_tiles` = batches x tiles of the chosen size (g.tiles_m, g.tiles_n set for it).  The caller has checked what the
// direct loads need (pitches, an MN-major extent divisible by 4, K % 4 == 0 for a K-major operand when K is no multiple
// of 16) and N <= 2^22.  false: no such variant.
// (64x64: a ring of eight stages, for long reductions over few tiles)
enum PanelTile : int { PANEL_TILE_128x128 = 0, PANEL_TILE_64x64 = 1 };
bool launch_gemm_panel(const GemmArgs& g, int tile, int amode, int bmode, unsigned cus, unsigned total_tiles, bool by_batch, hipStream_t stream);

// A small left operand against a very wide right one (one matrix, K up to 256, B with unit stride along N, plain store):
// persistent workgroups that keep their tile row of A in LDS and stream B alone (gemm_resident.hip).  `bm`: 128 (one
// workgroup per CU) or 64 (two) rows per tile, 64 columns; g.tiles_m, g.tiles_n set for that tile; the number of tile
// rows must not exceed the workgroups of an XCD.  The caller has checked what the direct loads need, as for the K-stream
// kernel.  false: not a shape this kernel takes.
bool launch_gemm_resident(const GemmArgs& g, int bm, int amode, int bmode, unsigned cus, hipStream_t stream);

} // namespace tenmo
