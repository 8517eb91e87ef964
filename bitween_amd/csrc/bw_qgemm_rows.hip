// bw_qgemm_rows.hip - the 64-row and the 256-row output tiles of the prefill kernel (natural-order schedule), in a
// translation unit of their own so that they compile beside the 128-row instantiations of bw_qgemm.hip.
//   64 rows  (a wave owns 64 x 64, 64 accumulation registers): calls of at most 64 rows - half the MFMAs and half the
//            activation traffic of a 128-row tile that would be at least half padding; two workgroups fit a CU
//   256 rows (a wave owns 256 x 64, all 256 accumulation registers): grids that fill the device - every weight is
//            unpacked once for twice the rows
// Which height a call gets is decided in bw_qgemm.hip (gemm_tile_rows).
#include "bw_qgemm_kernel.h"

int bw_launch_gemm_rows(int bits, int group, int rows, const GemmArgs& a, void* workspace, size_t workspace_bytes, hipStream_t stream) {
#define BW_CASE(B, G)                                                                                \
    if (bits == B && group == G)                                                                      \
        return rows == 256 ? launch_gemm<B, G, 16, true>(a, workspace, workspace_bytes, stream)       \
             : rows == 64  ? launch_gemm<B, G, 4, true>(a, workspace, workspace_bytes, stream)        \
                           : BW_EUNSUPPORTED;
    BW_CASE(4, 128) BW_CASE(4, 64) BW_CASE(4, 32)
    BW_CASE(8, 128) BW_CASE(8, 64) BW_CASE(8, 32)
    BW_CASE(2, 128) BW_CASE(2, 64) BW_CASE(2, 32)
#undef BW_CASE
    return BW_EUNSUPPORTED;
}
