/*
 * mmbo_gemm.h -- C ABI of the MI355X (gfx950) SGEMM/HGEMM/DGEMM library.
 *
 * Plain C: pointers, sizes and status codes only.  Every entry point names the piece of
 * the reference harness (CSWater/GEMM_MMBO, paths relative to its tree) that it replaces.
 *
 * Conventions shared by all GEMM entry points (reference: src/gemm/ref/Kernels.cpp:76-78,84-87,
 * src/gemm/gemm.h:4-5,28-40):
 *   - column-major storage:  op(A) is m x k, op(B) is k x n, C is m x n;
 *       transA == N:  A[i + l*lda]      transA == T:  A[l + i*lda]
 *       transB == N:  B[l + j*ldb]      transB == T:  B[j + l*ldb]
 *       C[i + j*ldc]
 *   - C = alpha * op(A) * op(B) + beta * C;  when beta == 0, C is never read
 *     (it may hold NaN or Inf) -- src/gemm/ref/Kernels.cpp:87;
 *   - A, B, C are DEVICE pointers owned by the caller (src/gemm/test.cc:53-66);
 *     alpha and beta are HOST pointers read before the call returns (src/gemm/gemm.h:31-32);
 *   - MMBO_F32: float A, B, C, alpha, beta; fp32 MFMA accumulate.
 *     MMBO_F16: IEEE binary16 A, B, C; alpha and beta are float; fp32 MFMA accumulate,
 *     one round-to-nearest-even to binary16 on the store.
 *     MMBO_F64: double A, B, C, alpha, beta (the reference's own element type); fp64 MFMA accumulate;
 *   - the launch is asynchronous on `stream` (a hipStream_t, NULL = the null stream the
 *     reference uses, src/gemm/common.h:12); the caller synchronises.  Configs with GlobalSplitU > 1 keep their
 *     partial sums in a workspace the library owns, one per (device, stream): GEMMs on different streams never
 *     share one, and calls from several host threads are safe.  A workspace is allocated on the first split-K call
 *     on its stream and grown when a call needs more (this waits for that stream's earlier work);
 *   - config_id selects a row of the tile-config table, like the reference's kernelId
 *     (src/gemm/constants.h:34-47,106-135); MMBO_CONFIG_AUTO lets the per-shape table pick.  Every shape runs
 *     under MMBO_CONFIG_AUTO.  Named configs: the general kernel's (no "DTL1" in the name) take any shape and
 *     alignment; of the direct-to-LDS ones ("DTL1") the "MFMA16x16" family takes m, n that end inside a tile, k that
 *     ends inside a slice and A, B at any element alignment (the reference's kernels take whole tiles only: its
 *     launcher floors the grid, src/gemm/driver.h:49-50), and reads no byte outside the operands: it fetches 16
 *     bytes at a time, and where m (transA = N) or n (transB = T) is not a whole number of such groups the last
 *     group of a column is the 16 bytes that end at its last element (refused, MMBO_ERR_INVALID_CONFIG, where that
 *     dimension is shorter than one group: 4 floats, 8 halves); the others need whole tiles and A, B, their
 *     leading dimensions and batch strides 16-byte aligned;
 *   - errors come back as status codes; nothing calls exit() (the reference's HIP_CHECK
 *     does, src/gemm/common.h:20-24).
 */
#ifndef MMBO_GEMM_H
#define MMBO_GEMM_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MMBO_F32 0
#define MMBO_F16 1
#define MMBO_F64 2

#define MMBO_OP_N 0
#define MMBO_OP_T 1

#define MMBO_CONFIG_AUTO (-1)

typedef enum mmbo_status {
    MMBO_OK = 0,
    MMBO_ERR_INVALID_DTYPE = 1,
    MMBO_ERR_INVALID_OP = 2,
    MMBO_ERR_INVALID_SIZE = 3,      /* ld too small, negative batch, dimension beyond 2^31-1 */
    MMBO_ERR_NULL_POINTER = 4,
    MMBO_ERR_INVALID_CONFIG = 5,    /* config_id outside the table, or not usable for this call */
    MMBO_ERR_HIP = 6,               /* a HIP runtime call failed; mmbo_last_hip_error() has the code */
    MMBO_ERR_NO_DEVICE = 7,         /* no gfx950 device is current */
    MMBO_ERR_WORKSPACE = 8          /* split-K workspace could not be allocated, or the partial sums of this call do
                                       not fit the static workspace of the entry point that allocates nothing */
} mmbo_status;

/* One row of the tile-config table (reference: the {MT0I, MT1J, threads} triples of
 * src/gemm/constants.h:34-47 and the solution dumps of src/gemm/ref/vega20_Cijk_Ailk_Bjlk_DB.yaml). */
typedef struct mmbo_config_desc {
    char name[64];          /* e.g. "MT256x256x64_WT128x064_W8_SK1"                       */
    int macro_tile_m;       /* MT0I: rows of C per work-group                              */
    int macro_tile_n;       /* MT1J: columns of C per work-group                           */
    int depth_u;            /* DepthU: k extent of one LDS stage                           */
    int threads;            /* work-group size (multiple of 64)                            */
    int wave_tile_m;        /* rows of C per wavefront (the MFMA-era "thread tile")        */
    int wave_tile_n;        /* columns of C per wavefront                                  */
    int split_k;            /* GlobalSplitU: 1 = none; >1 = partial sums + deterministic reduce */
    int lds_bytes;          /* LDS per work-group, worst case over the four transposes     */
} mmbo_config_desc;

/* GEMM.  Replaces naive_dgemm() / dgemm_NT() + launchGemm()
 * (src/gemm/gemm.h:4-45,47-97, src/gemm/driver.h:15-61): same argument meaning and order
 * (m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId), with the element type and the two
 * transposes made parameters instead of being baked into the function and kernel names. */
int mmbo_gemm(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
              const void *alpha, const void *A, size_t lda, const void *B, size_t ldb,
              const void *beta, void *C, size_t ldc, int config_id, void *stream);

/* Strided-batched GEMM: batch b uses A + b*strideA, B + b*strideB, C + b*strideC (strides in
 * elements).  The reference has no host API for it, but its kernel ABI carries the batch index
 * (sizeK, strideA2K/strideB2K/strideC2K in src/gemm/gemm.h:61-69,82-89; wgK = group_id(2) in
 * src/gemm/ref/Kernels.cpp:254); this is that capability exposed. */
int mmbo_gemm_strided_batched(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
                              const void *alpha, const void *A, size_t lda, long long strideA,
                              const void *B, size_t ldb, long long strideB,
                              const void *beta, void *C, size_t ldc, long long strideC,
                              int batch, int config_id, void *stream);

/* Tile-config table access.  Replaces indexing the parallel arrays of src/gemm/constants.h
 * and the NUM_KERNELS sweep bound of src/gemm/benchmark.cc:10,89-109.  Each element type has its own
 * table: ids are only meaningful together with the dtype they were asked for. */
int mmbo_num_configs(int dtype);
int mmbo_config_info(int dtype, int config_id, mmbo_config_desc *out);

/* The per-shape pick (reference: the exact-size -> solution table of
 * src/gemm/ref/vega20_Cijk_Ailk_Bjlk_DB.yaml:929-1177).  Returns a config id >= 0, or a
 * negative mmbo_status on bad arguments.  Pure host logic: needs no device. */
int mmbo_select_config(int dtype, int transA, int transB, size_t m, size_t n, size_t k, int batch);

/* Host twin of the kernels' work-group -> tile mapping: linear work-group id to (tile row, tile
 * column).  With num_xcd = 1 and linear_id = wg0 + wg1*nwg0 this is the reference's
 * WorkGroupMapping remap (src/gemm/ref/Kernels.cpp:204-236, src/gemm/ref/map.cpp:11-38);
 * num_xcd = 8 first regroups the round-robin XCD dispatch order so each XCD owns a contiguous
 * run of ids.  Pure host logic. */
int mmbo_wg_remap(unsigned linear_id, unsigned nwg0, unsigned nwg1, unsigned wgm, unsigned num_xcd,
                  unsigned *wg0, unsigned *wg1);

/* Host twin of the order in which the tiles that run one work-group per CU (256 x 256, 192 x 192, 256 x 192, 192 x 256 of
 * the 16x16-block kernel) are walked on grids of at least 16 x 16 tiles: chip-wide
 * blocks of 16 x 16 tiles (one per CU at a time), each XCD (linear_id % 8) on a 4 x 8 sub-block, blocks in
 * serpentine order, so the operand panels in flight at one time fit the last-level cache.  The reference maps
 * work-groups for its one L2 only (src/gemm/ref/Kernels.cpp:204-236); this is that idea one cache level up.
 * A bijection of [0, nwg0*nwg1); needs nwg0 >= 16 and nwg1 >= 16.  Pure host logic. */
int mmbo_chip_block_remap(unsigned linear_id, unsigned nwg0, unsigned nwg1, unsigned *wg0, unsigned *wg1);

/* Host twin of how a batch of small problems (at most 32 tiles each, batch a multiple of 8, no split-K) is laid over
 * the chip: linear dispatch index (tile slot + tiles * z, the order in which the hardware hands work-groups to its 8
 * XCDs round-robin) -> (tile, batch index), all tiles of one problem on one XCD so that the work-groups that read the
 * same panel of A or B share an L2.  The reference has no batches in its launcher (src/gemm/driver.h:49-59) and one
 * L2.  A bijection of [0, tiles*batch); needs batch % 8 == 0.  Pure host logic. */
int mmbo_batch_xcd_remap(unsigned linear_id, unsigned tiles, unsigned batch, unsigned *tile, unsigned *batch_index);

/* The same GEMM for callers that cannot allocate device memory -- code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose launcher allocates nothing either, but
 * has no split-K: GlobalSplitU 1, src/gemm/ref/vega20_Cijk_Ailk_Bjlk_DB.yaml:69).  Arguments, results and status codes
 * are those of mmbo_gemm_strided_batched (batch = 1 with zero strides is mmbo_gemm); the results are the same bit for bit.
 * The difference: the partial sums of a config with GlobalSplitU > 1 live in an array that is part
 * of the library's device image (mmbo_static_workspace_bytes() bytes of partial sums, 32 MiB, held by every GPU the
 * library runs on until the process ends) instead of in memory from hipMalloc, and the call makes no hipMalloc, hipFree
 * or other allocating call.  A call whose partial sums (GlobalSplitU x batch x m x n x 4 bytes; mmbo_config_info of
 * mmbo_select_config's pick gives GlobalSplitU) do not fit is refused with MMBO_ERR_WORKSPACE and launches nothing
 * when the caller named the config; under MMBO_CONFIG_AUTO the picked tile then runs with the largest GlobalSplitU
 * whose partial sums fit (down to none), so every shape runs under MMBO_CONFIG_AUTO here as well;
 * configs without split-K need no workspace and always run.  All calls on one GPU share that GPU's array: two such
 * split-K calls that overlap in time on one GPU (different streams, or different host threads) race on it -- keep them
 * on one stream.  The first call on a device looks the array's address up (hipGetSymbolAddress), once. */
int mmbo_gemm_strided_batched_static_workspace(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
                                               const void *alpha, const void *A, size_t lda, long long strideA,
                                               const void *B, size_t ldb, long long strideB,
                                               const void *beta, void *C, size_t ldc, long long strideC,
                                               int batch, int config_id, void *stream);
size_t mmbo_static_workspace_bytes(void);

/* Release the split-K workspaces held for the current device (one per stream that ran a split-K config; allocated
 * lazily, grown on demand, reused across calls).  Waits for the device.  The reference never frees what it loads
 * (src/gemm/driver.h:41).
 * The library keeps at most 8 such workspaces per device: a split-K call on a ninth stream retires the least recently
 * used one (it then waits for the device once).  A workspace is keyed by the stream handle and by the device that is
 * current at the call (make the stream's device current, as for any launch). */
int mmbo_release_workspace(void);

/* Release the workspace of one stream of the current device; waits for that stream only.  Call it before destroying
 * a stream that ran split-K configs when the memory should come back at once (otherwise the slot is retired when eight
 * other streams have needed one, or by mmbo_release_workspace).  A stream without a workspace is not an error. */
int mmbo_release_stream_workspace(void *stream);

/* How many split-K workspaces the library holds for the current device, and their total bytes (either pointer may
 * be null).  A diagnostic; no counterpart in the reference. */
int mmbo_workspace_info(size_t *slots, size_t *bytes);

/* Measures what the MFMA pipes of the current device sustain with nothing else running: a register-only loop
 * of v_mfma_f32_16x16x32_f16 (MMBO_F16), v_mfma_f32_32x32x2_f32 (MMBO_F32) or v_mfma_f64_16x16x4_f64 (MMBO_F64) -- the
 * instructions of the three fast paths --,
 * two wavefronts per SIMD, operands
 * all 1.0 (random_operands = 0) or uniform random (1).  Returns TFLOP/s and the average shader clock in MHz.
 * Counterpart of the reference's issue-only probe kernel src/gemm/assembly/error_kernel_000.s and of the
 * hard-coded 6.5 TFLOP/s peak its harness divides by (src/gemm/test.cc:88).  Allocates and frees a few
 * hundred KB; takes some tens of milliseconds. */
int mmbo_probe_mfma_ceiling(int dtype, int random_operands, double *tflops, double *shader_mhz);

/* Measures what a plain streaming kernel sustains on the current device with the byte counts of a memory-bound GEMM:
 * read_bytes read from one buffer and write_bytes written per launch (multiples of 16; either may be 0) -- to a second
 * buffer, or, with in_place set, over the first write_bytes of what was read, the way beta != 0 updates C --,
 * whole-chip grid-stride loops, `launches` launches back to back, the fastest of five such groups.  Returns seconds
 * per launch: the measured counterpart of the nominal 8 TB/s for shapes whose bound is memory (the batched and the
 * skinny benchmark configs), as mmbo_probe_mfma_ceiling is of the nominal matrix peak.  Buffers of up to a few hundred
 * MB stay in the last-level cache from launch to launch, as a GEMM's operands do in a benchmark loop.  The reference has
 * no bandwidth figure at all (its harness reports GFLOP/s against a hard-coded peak, src/gemm/test.cc:87-88).
 * Allocates and frees read_bytes + write_bytes. */
int mmbo_probe_stream(size_t read_bytes, size_t write_bytes, int in_place, int launches, double *seconds_per_launch);

const char *mmbo_status_string(int status);
int mmbo_last_hip_error(void);       /* hipError_t of the last MMBO_ERR_HIP on this thread */
const char *mmbo_version(void);

#ifdef __cplusplus
}
#endif
#endif
