/* C ABI of the dense fp16 GEMM with a stream-K tail in libmarlin_amd.so (gfx950).
 *
 * The reference's gemm/streamk_gemm is a stand-alone program without a library
 * interface: gemm_streamk.cu:8-110 builds A (m x k, row-major), B (k x n,
 * column-major, i.e. n rows of k) and C (m x n, row-major) in fp16 with
 * alpha = 1, beta = 0, fills an Arguments object (gemm_streamk.h, with the tile
 * split of dp_sk_block.h:31-128), allocates its workspace (init_workspace) and
 * launches gemmTN_streamk_dp.  streamk_gemm_tn stands for that sequence: the
 * caller passes the three device buffers and the sizes; the split, the
 * workspace and the launch are the library's.
 */
#ifndef STREAMK_AMD_H
#define STREAMK_AMD_H

#ifdef __cplusplus
extern "C" {
#endif

#define STREAMK_OK 0
#define STREAMK_ERR_SHAPE 1   /* negative size, n not a multiple of 256, k not a multiple of 64 */
#define STREAMK_ERR_RUNTIME 3 /* HIP error or size limit; text in streamk_amd_last_error() */

/* C = A * B^T on `hip_stream` (a hipStream_t) of device `dev`; asynchronous.
 * A: m x k fp16, row-major.  B: n x k fp16, row-major (the k x n column-major
 * operand of gemm_streamk.cu:29).  C: m x n fp16, row-major, written once.
 * fp32 accumulation.  m is arbitrary; n % 256 == 0 and k % 64 == 0.
 * Partial sums of the stream-K tiles live in the library-owned buffer of this
 * (device, stream) that marlin_gemm uses too (include/marlin_amd.h): sized by
 * the launch (tile rows x tile columns x 4 bytes per slice of a stream-K tile), grown on demand, none for
 * launches without stream-K tiles.  Calls on one stream may follow each other
 * freely, calls that overlap must use different streams; a call that would have
 * to allocate under graph capture returns STREAMK_ERR_RUNTIME. */
int streamk_gemm_tn(const void* A, const void* B, void* C, int m, int n, int k, int dev,
                    void* hip_stream);

/* return code streamk_gemm_tn would give for these sizes (no GPU touched) */
int streamk_amd_check(int m, int n, int k);

/* the tile split for a device with `cus` compute units (counterpart of
 * SK_DP_Block_Wrapper, dp_sk_block.h:31-80): out[0..7] = tiles along m, tiles
 * along n (tiles numbered in panels of 8 column tiles), data-parallel tiles, stream-K
 * tiles (the last ones in tile order), k slices per stream-K tile, workgroups,
 * rows of a tile (256, or 128 when 256 x 256 tiles would occupy at most half
 * of the compute units), columns of a tile (256, or 128 when 128 x 256 tiles
 * would occupy at most half of them too) */
int streamk_amd_plan(int m, int n, int k, int cus, int* out);

/* out[0], out[1] = row and column tile of tile number `tile` (0 <= tile <
 * tiles_m * tiles_n); for tests of the numbering */
void streamk_amd_tile_coord(int tile, int tiles_m, int tiles_n, int* out);

/* same as marlin_amd_release (include/marlin_amd.h): frees the partial-sum
 * buffers of device dev (all if dev < 0), returns the bytes freed */
long long streamk_amd_release(int dev);

/* text of the last STREAMK_ERR_RUNTIME on this thread */
const char* streamk_amd_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
