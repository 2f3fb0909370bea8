/*
 * webdnn_hip.h — C ABI of libwebdnn_hip.so, the native side of the `hip`
 * backend for the WebDNN descriptor runner.
 *
 * The reference has no C header for this path: its native precedent is the
 * WASM worker protocol (integer buffer ids + `extern "C"` kernels taking raw
 * float pointers and int/float scalars):
 *   src/descriptor_runner/backend/wasm/wasmContextImpl.ts:113-163
 *       (alloc / destroy / write / read / runKernel messages)
 *   src/shader/wasm/pre.js:4-91            (id -> pointer table, dispatch)
 *   src/shader/wasm/src/core/allocation.cpp:4-15   (webdnn_malloc/free)
 *   src/shader/wasm/src/kernels/standard/gemm.cpp:19-104 (kernel_gemm_*)
 * Each entry point below names the reference interface it stands in for.
 *
 * Conventions
 *   - every function returns 0 on success and a negative WDH_E* code on
 *     failure; it never aborts or throws.  wdh_last_error() returns a
 *     message for the last failure on the calling thread.
 *   - device buffers are named by opaque positive 64-bit handles
 *     (wdh_alloc); 0 means "no tensor" where a tensor is optional.
 *   - all work is enqueued on ONE HIP stream owned by the library; calls
 *     return as soon as the work is enqueued.  wdh_read() and wdh_sync()
 *     are the only blocking calls.
 *   - all tensors are dense row-major; float tensors are IEEE fp32,
 *     index tensors int32 (the runner clips ONNX int64 to int32:
 *     src/descriptor_runner/core/runnerImpl.ts:167-198).
 *   - strides are in ELEMENTS, not bytes.
 *   - the library is not re-entrant: call it from one thread at a time
 *     (the descriptor runner is single-threaded:
 *     src/descriptor_runner/core/runnerImpl.ts:377-542).
 */
#ifndef WEBDNN_HIP_H_
#define WEBDNN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WDH_OK 0
#define WDH_ENODEV (-1)   /* no usable gfx950 device / driver            */
#define WDH_EINVAL (-2)   /* bad argument (shape, handle, stride, op id) */
#define WDH_ENOMEM (-3)   /* device or pinned-host allocation failed     */
#define WDH_EHIP (-4)     /* a HIP runtime call failed                   */
#define WDH_ESTATE (-5)   /* library not initialised                     */

typedef int64_t wdh_buf;

/* ---- lifetime -------------------------------------------------------- */

/* Replaces WebDNNWasmContextImpl.initialize() (worker start-up),
 * backend/wasm/wasmContextImpl.ts:39-73.  Selects `device`, creates the
 * stream, the pinned staging buffers and the buffer pool.  WDH_ENODEV when
 * there is no device: the host context must turn that into a thrown Error so
 * that load() skips the backend (src/descriptor_runner/index.ts:68-79). */
int wdh_init(int device);
void wdh_shutdown(void);
/* Message for the most recent failure on this thread ("" if none). */
const char *wdh_last_error(void);
/* Device facts used for roofline arithmetic (name is NUL-terminated). */
int wdh_device_info(char *name, int name_cap, int *compute_units,
                    int *clock_mhz, uint64_t *hbm_bytes);

/* Backend options (the counterpart of InitOption.backendOptions,
 * src/descriptor_runner/index.ts:26-30).  Known names:
 *   "contraction_tile"  -1 = choose per problem (default); 0 = 128x128,
 *                       1 = 64x256, 2 = 64x128, 3 = 64x64, 4 = 128x64 workgroup tiles for
 *                       wdh_gemm / wdh_conv2d (a tuning and test hook: every
 *                       tile shape computes the same result).
 *   "split_k"           -1 = choose per problem (default); n >= 1 = cut the
 *                       K loop of every tile of wdh_gemm / wdh_conv2d into n
 *                       chunks whose partial sums are added in chunk order
 *                       by a second kernel (1 = never split).
 *   "conv3x3_halo"      1 (default) = 3x3, stride-1, undilated convolutions whose
 *                       input channels per group are a multiple of 8 stage the
 *                       input rows of a tile in LDS and read the taps from there;
 *                       0 = they gather taps from global memory like every other
 *                       geometry (both forms compute the same sums).
 *   "conv3x3_winograd"  how 3x3, stride-1, undilated, ungrouped convolutions whose channel count is a
 *                       multiple of 16 are computed: 1 (default) = those with at least 128 input and
 *                       128 output channels by the minimal-filtering algorithm F(2x2, 3x3) (filters
 *                       and 4x4 input patches transformed, 16 batched matrix products with 4/9 of
 *                       the multiplications, results transformed back under the epilogue; rounding
 *                       errors like the direct form's, about 1.5e-7 of max|ref|); 2 = all of them
 *                       that way; 3 = all of them by F(4x4, 3x3) (6x6 patches, 36 products, a quarter
 *                       of the multiplications; 10-20 % faster than F(2x2, 3x3) from 64 channels on,
 *                       rounding errors about 1e-6 of max|ref|: inside the Gemm/Conv tolerance, but
 *                       ResNet-50's logits then differ from the CPU path's by 1.7e-3 where 1e-3 is
 *                       asked and the other forms give 7e-4); 0 = none (the direct forms below).
 *                       Not the direct form's sums: no form agrees with another bit for bit.
 *   "conv3x3_f4x4_channels"  0 (default) or a channel count from which "conv3x3_winograd" 1 takes
 *                       F(4x4, 3x3) instead (64 is where it starts to win): for callers who can
 *                       trade the last digit for speed.
 *   "memory_limit_mib"  0 (default) = no limit, or the most device memory, in MiB, that the buffer pool
 *                       asks the driver for: an allocation beyond it first gives cached blocks back, then
 *                       fails with WDH_ENOMEM.  Workspaces are subject to it: a conv that cannot get
 *                       the tensors of its minimal-filtering form takes a direct form instead.
 *   "conv_stem"         1 (default) = a 7x7, stride-2, undilated convolution from 3 to 64
 *                       channels (the stem of an image network) runs in a kernel that keeps
 *                       all weights and a tile's input patch in LDS; 0 = it gathers taps
 *                       from global memory like every other geometry (same sums, added
 *                       in another order).
 *   "gemm_wavesplit"    1 (default) = a Gemm / MatMul with few result tiles and K >= 128
 *                       runs as one launch of 32x32 blocks whose 16 wavefronts share K
 *                       among themselves; 0 = it takes the ordinary tiles (K cut across
 *                       workgroups, partial sums added by a second kernel).
 *   "wide_stores"       1 (default) = whole result tiles whose rows are 16-byte aligned
 *                       (Conv: output planes of a multiple of four pixels; Gemm: row and
 *                       batch strides of Y that are multiples of four) are turned through
 *                       LDS and stored 16 bytes per lane; 0 = every lane stores single
 *                       elements (same arithmetic, same bits).
 *   "conv1x1_stride2_in_place"  1 (default) = an unpadded 1x1 convolution with a column stride of
 *                       2 whose output rows hold an even number of pixels (input rows a multiple
 *                       of four) reads X in place (16-byte pieces, every other element kept); 0 = it gathers its
 *                       taps from global memory like every other strided geometry.
 *   "stream_k"          how wdh_gemm / wdh_conv2d launches whose tiles do not fill the chip in
 *                       whole rounds are scheduled: 1 (default) = such launches keep a fixed
 *                       grid of resident workgroups, each of which multiplies an equal,
 *                       contiguous share of all K slabs of the launch, tile borders or not;
 *                       a tile shared by neighbouring workgroups is added up in K order by
 *                       the one that holds its last slabs (one launch, no second pass);
 *                       2 = every launch that can; 0 = none (one tile or K chunk per
 *                       workgroup, chunks added by a second kernel).  The sums of a tile are
 *                       added in another order than with 0; both orders are fixed.
 *   "stream_wgs"        1..8 (default 4) = resident workgroups per CU of such a launch.
 *   "stream_spin"       how often a workgroup polls for a neighbour's partial tile before it
 *                       gives up (the next wdh_sync / wdh_read then fails with WDH_EHIP); a
 *                       test hook.
 *   "descriptor_loads"  1 (default) = operands below 2 GiB are read and written
 *                       through buffer descriptors with 32-bit offsets; 0 = every
 *                       operand is treated as if it spanned 2 GiB or more (64-bit
 *                       addresses, bounds-checked stores, the gather form for every
 *                       convolution).  A test hook: it runs the large-operand code
 *                       on ordinary sizes. */
int wdh_set_option(const char *name, int value);
/* wdh_init also applies the options named in the environment variable WDH_OPTIONS
 * ("name=value,name=value"), for hosts that cannot call wdh_set_option themselves. */

/* How the most recent wdh_gemm / wdh_conv2d launch was laid out (for per-layer
 * reports; cf. the per-node records of measurePerformance,
 * core/runnerImpl.ts:533-541): workgroup tile, the number of tiles computed whole
 * and of tiles cut along K, chunks per cut tile (1 = none), and which form of the
 * kernel ran: WDH_FORM_* below.  A launch scheduled as a stream of K slabs ("stream_k")
 * reports split = 0, all its tiles as whole_tiles and its workgroup count as split_tiles.
 * Any pointer may be NULL. */
#define WDH_FORM_GEMM_KC 0        /* B k-contiguous (transB)                    */
#define WDH_FORM_GEMM_MC 1        /* B n-contiguous                             */
#define WDH_FORM_CONV_GATHER32 2  /* taps gathered from X, at most 31 taps      */
#define WDH_FORM_CONV_GATHER64 3  /* ... 32 to 63 taps                          */
#define WDH_FORM_CONV_GATHER_FLAT 4 /* ... more taps or X of 2 GiB or more      */
#define WDH_FORM_CONV_PIXELS 5    /* 1x1 stride 1: X read in place              */
#define WDH_FORM_CONV3X3_LDS 6    /* 3x3 stride 1: taps read from an LDS tile   */
#define WDH_FORM_CONV_STEM 7      /* 7x7 stride 2, 3 -> 64 channels: weights and the
                                   * input patch of an 8x16-pixel tile in LDS   */
#define WDH_FORM_CONV_PIXELS_S2 8 /* 1x1 with column stride 2: X read in place,
                                   * every other pixel of a row kept            */
#define WDH_FORM_CONV3X3_WINOGRAD 9 /* 3x3 stride 1 as F(2x2, 3x3): transforms around a
                                   * batched product (tile and split are the product's) */
#define WDH_FORM_CONV3X3_WINOGRAD4 10 /* ... as F(4x4, 3x3)                              */
int wdh_last_plan(int *tile_m, int *tile_n, int64_t *whole_tiles,
                  int64_t *split_tiles, int *split, int *form);

/* ---- buffers --------------------------------------------------------- */

/* Replaces the `alloc` message, wasmContextImpl.ts:128-134 and
 * webdnn_malloc, allocation.cpp:4-9.  Returns a handle > 0, or 0 on failure
 * (see wdh_last_error).  Zero-byte requests succeed.  Contents are
 * undefined.  Blocks come from a size-bucketed pool of hipMalloc memory. */
wdh_buf wdh_alloc(size_t bytes);
/* Replaces `destroy`, wasmContextImpl.ts:136-141.  The block returns to the
 * pool; work already enqueued on the stream still sees valid memory because
 * later users are ordered behind it on the same stream. */
int wdh_free(wdh_buf h);
/* Replaces `write`, wasmContextImpl.ts:143-151: host -> device through
 * pinned staging + hipMemcpyAsync.  `src` may be reused on return. */
int wdh_write(wdh_buf h, size_t dst_offset, const void *src, size_t bytes);
/* Replaces `read`, wasmContextImpl.ts:153-163: device -> host; blocks until
 * every previously enqueued kernel and this copy have finished. */
int wdh_read(wdh_buf h, size_t src_offset, void *dst, size_t bytes);
/* Device-to-device copy; replaces kernel_copy,
 * src/shader/wasm/src/kernels/standard/copy.cpp:6-8. */
int wdh_copy(wdh_buf dst, size_t dst_offset, wdh_buf src, size_t src_offset,
             size_t bytes);
/* Waits for the work of the current lane (see wdh_set_lane). */
int wdh_sync(void);

/* Lanes: several runs in flight.  No counterpart in the reference (its backends run one graph at a time);
 * for callers that keep a second batch on its way while the first computes.  A lane is a HIP stream of
 * default priority; lane 0 is the stream everything runs on unless told otherwise, lanes 1 .. WDH_LANES - 1
 * are side lanes, created when first named.  wdh_set_lane(1) makes lane 1 the current one: wdh_write, wdh_read, wdh_copy, wdh_sync, wdh_event_record,
 * wdh_graph_begin / _end / _launch then work on it, concurrently with what lane 0 still has queued.
 * Side lanes are for captured runs and their transfers: an operator call (wdh_gemm, wdh_conv2d, ...) on
 * a side lane is legal only while a graph is being recorded there and fails with WDH_ESTATE otherwise.
 * What the library guards by itself: a block freed while a side lane has work in flight waits for that
 * lane first; an allocation or a capture on a side lane waits for lane 0; launches that run as streams
 * of K slabs use a workspace of the lane's own (WDH_STATIC_SCRATCH_BYTES from the driver when the lane is
 * first used), so a run recorded on a side lane computes bit for bit what it computes on lane 0;
 * wdh_gemm_static is refused there (its workspace is lane 0's); a wdh_copy on a side lane first waits
 * for uploads (wdh_write) still on their way on any lane.  A recorded run may be launched on any lane, but it
 * keeps using the stream workspace of the lane it was recorded on: launch two recordings at the same time
 * only if they were made on different lanes (runner.submit does).  What the caller guards: a buffer written on one lane and read on another needs a
 * wdh_sync (or wdh_read) on the first in between.  Not possible while capturing. */
#define WDH_LANES 4
int wdh_set_lane(int lane);

/* Side branches of a recorded run.  No counterpart in the reference.  Between wdh_graph_begin and
 * wdh_graph_end, the calls made between wdh_branch_begin and wdh_branch_end are recorded as a branch that
 * depends only on what was recorded before wdh_branch_begin; the calls after wdh_branch_end do not depend
 * on the branch until wdh_branch_join, so a replay may run the branch next to them (a projection shortcut
 * next to the convolutions it bypasses).  One branch at a time.  The caller promises that nothing recorded
 * between _end and _join reads what the branch writes or writes what it reads.  The library keeps the
 * buffers apart: a block freed while a branch is open is handed out again only after the join, and no
 * launch takes the stream-of-K-slabs form while one is open (that form's workspace is one per lane).
 * Outside a recording the three calls do nothing: the work simply runs in the order of the calls, with the
 * same results bit for bit.  wdh_graph_end joins a branch that was left open. */
int wdh_branch_begin(void);
int wdh_branch_end(void);
int wdh_branch_join(void);

/* Pool accounting: bytes handed out, bytes cached in the pool, high-water
 * mark of hipMalloc'ed bytes (cf. perfTotalMemory,
 * backend/wasm/wasmTensorImpl.ts:29-35).  Any pointer may be NULL. */
int wdh_mem_stats(uint64_t *in_use, uint64_t *cached, uint64_t *peak);
/* Return cached blocks to the driver (cf. deallocateToBytes,
 * backend/webgl/webglContextImpl.ts:541-568). */
int wdh_trim(size_t keep_bytes);

/* ---- captured runs --------------------------------------------------------
 * The reference runs its node loop in JavaScript on every RunnerImpl.run
 * (core/runnerImpl.ts:377-542); here the device work of one run can be recorded
 * once into a HIP graph and replayed with a single launch.
 * Between wdh_graph_begin and wdh_graph_end every operator entry point, wdh_copy,
 * wdh_alloc and wdh_free records instead of executing; blocks allocated meanwhile
 * become the graph's own memory (recycled among its tensors, lent to nobody else)
 * until wdh_graph_destroy.  Calls that need the host to see device data or the
 * stream to drain (wdh_write, wdh_read, wdh_sync, wdh_trim, events, the first
 * wdh_conv2d of a geometry) fail with WDH_ESTATE and make wdh_graph_end fail:
 * run the model once eagerly first.  Buffers that exist before the capture
 * (weights, inputs) and handles still held after it (outputs) are what a replay
 * reads and writes: refill the inputs with wdh_write, call wdh_graph_launch, read
 * the outputs with wdh_read. */
int wdh_graph_begin(void);
int wdh_graph_end(int *graph_id);
int wdh_graph_launch(int graph_id);
int wdh_graph_destroy(int graph_id);

/* ---- timing (measurePerformance, core/runnerImpl.ts:368-375,533-541) -- */

#define WDH_MAX_EVENTS 4096
int wdh_event_record(int id);              /* 0 <= id < WDH_MAX_EVENTS */
int wdh_event_elapsed_ms(int start_id, int stop_id, float *ms); /* blocks */

/* ---- epilogues shared by gemm / conv ---------------------------------- */

#define WDH_EPI_NONE 0
#define WDH_EPI_RELU 1      /* y = max(y, 0) with Math.max semantics      */

/* ---- Gemm / MatMul ----------------------------------------------------
 * Replaces CpuGemm.run (operators/cpu/operators/standard/gemm.ts:21-61),
 * CpuMatMul.calcDim2/calcDim3 (.../matmul.ts:58-111) and the WASM
 * kernel_gemm_transa{0,1}_transb{0,1}[_c] family (gemm.cpp:19-104).
 *
 *   for b < batch, i < m, j < n:
 *     acc          = sum_{x<k} A[b*sAb + i*sA0 + x*sA1] * B[b*sBb + x*sB0 + j*sB1]
 *     Y[(b*m+i)*n+j] = epi( f32(alpha*acc) + beta * C[i*sC0 + j*sC1] )
 *
 * C == 0 means no C term (MatMul; Gemm without bias).  sC0/sC1 come from the
 * unidirectional broadcast of C to [m,n] (operatorUtil.ts:178-209), so either
 * may be 0.  sAb/sBb may be 0 (batch broadcast, base/matmul.ts:60-70).
 * transA/transB are expressed through the strides exactly as
 * base/gemm.ts:39-56 does.  At least one of (sA0,sA1) and one of (sB0,sB1)
 * must be 1 or the extent along it 1 (dense operands).
 * `R` (0 = none) is an optional residual of shape [batch,m,n] added after the
 * C term and before the epilogue; it exists for fused MatMul+Add graphs. */
int wdh_gemm(wdh_buf A, wdh_buf B, wdh_buf C, wdh_buf Y, int batch, int m,
             int n, int k, int64_t sAb, int64_t sA0, int64_t sA1, int64_t sBb,
             int64_t sB0, int64_t sB1, int64_t sC0, int64_t sC1, float alpha,
             float beta, int epilogue, wdh_buf R);

/* wdh_gemm with a spaced-out result: Y[b, i, j] = Y[b*sYb + i*sY0 + j] (R alike), rows
 * contiguous.  It lets a MatMul write straight into the layout a following Transpose
 * would have produced (attention heads merged back: [heads, tokens, d] stored as
 * [tokens, heads, d], CPUTranspose.copyNd, transpose.ts:46-168, absorbed into the
 * product).  wdh_gemm is this call with sYb = m*n, sY0 = n.  Batch entries must not
 * overlap: sYb >= m*sY0, or sYb >= n and sY0 >= batch*sYb. */
int wdh_gemm_ex(wdh_buf A, wdh_buf B, wdh_buf C, wdh_buf Y, int batch, int m,
                int n, int k, int64_t sAb, int64_t sA0, int64_t sA1, int64_t sBb,
                int64_t sB0, int64_t sB1, int64_t sC0, int64_t sC1, float alpha,
                float beta, int epilogue, wdh_buf R, int64_t sYb, int64_t sY0);

/* `count` (at most 16) independent linear layers Y_i[m_i, n_i] = A_i[m_i, k_i] W_i[k_i, n_i]
 * (+ bias_i[n_i]) (then Relu if `epilogue` is WDH_EPI_RELU), all operands dense and
 * row-major: each is exactly the wdh_gemm call of a MatMul node followed by its bias Add
 * (operators/cpu/operators/standard/matmul.ts:11-111, binary7.ts:24-75).  Products small
 * enough for the one-launch form of wdh_gemm (few 32x32 result blocks, K cut across the
 * wavefronts of a workgroup) leave together in one launch, which is what this entry point
 * is for: the query, key and value projections of an attention block are three such
 * products; the others are launched one by one as wdh_gemm would.  Results are the bits
 * wdh_gemm stores.  `bias` may be NULL, or hold 0 for a layer without bias; every Y_i
 * must be a buffer of its own that no problem of the group reads. */
int wdh_linear_group(int count, const wdh_buf *A, const wdh_buf *W, const wdh_buf *bias,
                     const wdh_buf *Y, const int *m, const int *n, const int *k, int epilogue);

/* wdh_gemm for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, same kernels and bit-identical
 * results as wdh_gemm; the one difference is where the partial sums of tiles cut
 * along K live: in a workspace of WDH_STATIC_SCRATCH_BYTES inside the library's
 * own device image (one copy per GPU, held until the process ends) instead of a
 * block from the pool.  The call performs no hipMalloc / hipFree and takes nothing
 * from the pool.  A problem whose plan needs more workspace than that fails with
 * WDH_EINVAL and touches nothing (wdh_set_option("split_k", 1) makes every size fit:
 * unsplit launches use no workspace).  All calls on a GPU share the one workspace,
 * which keeps the previous call's contents: the kernels write every partial sum
 * they later read, so nothing has to be cleared, but two such calls that overlap
 * on one GPU (other streams, other threads) race; lane 0, the only lane that takes
 * this call, orders them. */
#define WDH_STATIC_SCRATCH_BYTES ((32u << 20) + (160u << 10))
int wdh_gemm_static(wdh_buf A, wdh_buf B, wdh_buf C, wdh_buf Y, int batch, int m,
                    int n, int k, int64_t sAb, int64_t sA0, int64_t sA1,
                    int64_t sBb, int64_t sB0, int64_t sB1, int64_t sC0,
                    int64_t sC1, float alpha, float beta, int epilogue, wdh_buf R);

/* ---- Conv (2-D, NCHW) ------------------------------------------------
 * Replaces CpuConv.run = im2col + matmul + transpose + bias
 * (operators/cpu/operators/standard/conv.ts:134-333) and the four WebGPU
 * dispatches (operators/webgpu/operators/standard/conv.ts:13-120).
 *   X [n, c, h, w]   W [cout, c/group, kh, kw]   Bias [cout] or 0
 *   Y [n, cout, oh, ow],  oh = floor((h+pt+pb-dh*(kh-1)-1)/sh)+1 (base/conv.ts:43-59)
 *   Y = epi( f32(sum) + bias[co] (+ R) );  R: optional residual shaped like Y. */
int wdh_conv2d(wdh_buf X, wdh_buf W, wdh_buf Bias, wdh_buf Y, int n, int c,
               int h, int w, int cout, int kh, int kw, int pt, int pl, int pb,
               int pr, int sh, int sw, int dh, int dw, int group, int epilogue,
               wdh_buf R);
/* wdh_conv2d with promises about the operands.  WDH_CONV_CONSTANT_WEIGHTS: nobody writes to W
 * while its handle lives -- what holds for the device copy of an initializer, which the runner
 * uploads once and keeps across runs (copiedInitializerTensors, core/runnerImpl.ts:323-351).
 * The library may then keep data derived from W (the transformed filters of the F(2x2, 3x3)
 * form) from one call to the next; it is dropped when W is freed, written to through wdh_write
 * or wdh_copy, or at wdh_shutdown.  Results are those of wdh_conv2d. */
#define WDH_CONV_CONSTANT_WEIGHTS 1
int wdh_conv2d_ex(wdh_buf X, wdh_buf W, wdh_buf Bias, wdh_buf Y, int n, int c,
                  int h, int w, int cout, int kh, int kw, int pt, int pl, int pb,
                  int pr, int sh, int sw, int dh, int dw, int group, int epilogue,
                  wdh_buf R, int flags);

/* ---- elementwise -------------------------------------------------------
 * Replaces Binary7 (operators/cpu/operators/standard/binary7.ts:16-68) and
 * kernel_{add,sub,mul,div,pow}_d0..d6 (binary7s.cpp:9-22).  ndim <= 6;
 * strides come from broadcastMulti (operatorUtil.ts:211-245): 0 on broadcast
 * axes.  dtype: 0 = float32, 1 = int32 (Pow: float32 only here). */
#define WDH_BIN_ADD 0
#define WDH_BIN_SUB 1
#define WDH_BIN_MUL 2
#define WDH_BIN_DIV 3
#define WDH_BIN_POW 4
int wdh_binary(int op, int dtype, wdh_buf L, wdh_buf R, wdh_buf Y, int ndim,
               const int32_t *out_shape, const int64_t *strides_l,
               const int64_t *strides_r);

/* Replaces CPUUnary (operators/cpu/operators/standard/unary.ts:10-32) and
 * kernel_{relu,sigmoid,sqrt,exp,tanh,...} (unarys.cpp:11-17).
 * dtype 1 (int32) is accepted for RELU, ABS and NEG only. */
#define WDH_UN_RELU 0
#define WDH_UN_SIGMOID 1   /* (tanh(x/2)+1)/2, unary.ts:158-164 */
#define WDH_UN_SQRT 2
#define WDH_UN_EXP 3
#define WDH_UN_TANH 4
#define WDH_UN_ABS 5
#define WDH_UN_NEG 6
#define WDH_UN_RECIPROCAL 7
int wdh_unary(int op, int dtype, wdh_buf X, wdh_buf Y, size_t length);
/* Replaces Cast (operators/cpu/operators/standard/cast.ts:12-52): dtypes are
 * 0 = float32, 1 = int32 (the runner's two; ONNX INT64/UINT8 arrive as int32).
 * float32 -> int32 applies ToInt32 (what `Int32Array.set` does: truncate, wrap
 * modulo 2^32, NaN and infinities give 0); int32 -> float32 rounds to nearest. */
int wdh_cast(int from_dtype, int to_dtype, wdh_buf X, wdh_buf Y, size_t length);

/* ---- row reductions ----------------------------------------------------
 * Softmax over the last axis: X viewed as [outer, len]; replaces
 * Softmax.run (operators/cpu/operators/standard/softmax.ts:34-57). */
int wdh_softmax(wdh_buf X, wdh_buf Y, int64_t outer, int len);
/* softmax(alpha * Q K^T) V for `batch` heads in one launch: what the chain MatMul -> Mul
 * by a constant -> Softmax -> MatMul computes (operators/cpu/operators/standard/
 * matmul.ts:11-111, softmax.ts:34-57; the reference runs the four nodes one after the
 * other), with the rounding points of that chain.  Element (b, i, x) of Q is at
 * b*sQb + i*sQi + x, key j of K at b*sKb + j*sKj + x, of V at b*sVb + j*sVj + x and
 * result (b, i, x) at b*sYb + i*sYi + x: the head dimension d (32, 64 or 128) is the
 * contiguous one everywhere, which is how the heads lie in a [tokens, heads, d]
 * projection, so no Transpose of Q, K, V or of the result is needed.  At most 1024
 * keys (a 32 x keys block of scores is kept in LDS); Q and K 16-byte aligned with
 * strides that are multiples of 4; Y must not alias an input.  Anything else is
 * WDH_EINVAL: the caller runs the separate operators instead. */
int wdh_attention(wdh_buf Q, wdh_buf K, wdh_buf V, wdh_buf Y, int batch, int tq, int tk, int d,
                  int64_t sQb, int64_t sQi, int64_t sKb, int64_t sKj, int64_t sVb,
                  int64_t sVj, int64_t sYb, int64_t sYi, float alpha);
/* LayerNormalization over the last axis (ONNX opset 17, biased variance).
 * The reference has no such operator on any backend; this is what the
 * decomposed ReduceMean/Sub/Pow/Sqrt/Div/Mul/Add subgraph
 * (operators/cpu/operators/standard/reduce.ts:369-405 + binary7/unary)
 * computes.  Gamma/Beta are [len] or 0 (1 / 0 respectively). */
int wdh_layernorm(wdh_buf X, wdh_buf Gamma, wdh_buf Beta, wdh_buf Y,
                  int64_t outer, int len, float eps);
/* LayerNormalization followed by the Add that reads its result: Y as wdh_layernorm, and
 * Y2 = Y + P with P of X's shape (both results are kept: the graph reads the normalised rows
 * again later).  Replaces the node pair LayerNormalization -> Add (binary7.ts:24-75 for the
 * Add; the reference has no LayerNormalization); Y2 holds exactly what the separate Add
 * would store.  Y2 must not alias X, Y or P. */
int wdh_layernorm_add(wdh_buf X, wdh_buf Gamma, wdh_buf Beta, wdh_buf Y, wdh_buf P, wdh_buf Y2,
                      int64_t outer, int len, float eps);
/* ReduceMean over the trailing `len` elements of each of `outer` rows;
 * replaces ReduceMean (reduce.ts:369-405) for trailing-axes reductions. */
int wdh_reduce_mean(wdh_buf X, wdh_buf Y, int64_t outer, int len);
/* One pass of ReduceMean over an arbitrary set of axes: the reference reduces the
 * axes one after the other in ascending order (ReduceOp.runCore, reduce.ts:40-100),
 * each pass a sum in double stored as fp32, the last pass divided by the product of
 * all reduced extents (reduce.ts:369-405).  X viewed as [outer, red, inner]:
 *   Y[o, i] = f32( (sum_r X[o, r, i]) / divisor ),  divisor = 1 for all passes but the last. */
int wdh_reduce_axis(wdh_buf X, wdh_buf Y, int64_t outer, int red, int64_t inner,
                    int64_t divisor);

/* ---- pooling -------------------------------------------------------------
 * Replaces CpuMaxPool.maxpool (operators/cpu/operators/standard/maxpool.ts:58-112);
 * pads/out sizes come from MaxPool.calcShape (operators/base/maxpool.ts:32-137).
 * Cells outside the input are skipped; a window with no valid cell yields -inf. */
int wdh_maxpool2d(wdh_buf X, wdh_buf Y, int n, int c, int h, int w, int oh,
                  int ow, int kh, int kw, int pt, int pl, int sh, int sw,
                  int dh, int dw);
/* Replaces CpuGlobalAveragePool.run (globalaveragepool.ts:12-41) +
 * averagepool() (rawcomputation/averagepool.ts:1-46): Y[nc] = mean over hw. */
int wdh_global_avgpool(wdh_buf X, wdh_buf Y, int64_t nc, int hw);

/* ---- layout --------------------------------------------------------------
 * Replaces CPUTranspose.copyNd (operators/cpu/operators/standard/transpose.ts:46-168):
 * Y[dense index over out_shape] = X[sum_i idx_i * in_strides[i]];
 * ndim <= 6; elem_bytes must be 4. */
int wdh_transpose(wdh_buf X, wdh_buf Y, int ndim, const int32_t *out_shape,
                  const int64_t *in_strides);
/* Replaces Gather (operators/cpu/operators/standard/gather.ts:20-33), widened
 * to the general axis form: data viewed as [outer, axis_len, inner], int32
 * indices[n_idx] (negative indices wrap once) -> Y [outer, n_idx, inner]. */
int wdh_gather(wdh_buf Data, wdh_buf Indices, wdh_buf Y, int64_t outer,
               int axis_len, int64_t inner, int64_t n_idx);
/* Replaces the copy loops of Slice10.copy1d..copy6d
 * (operators/cpu/operators/standard/slice.ts:96-330), Concat.run
 * (concat.ts:21-84) and CPUSplit2/13.run (split.ts:12-87), which are all
 *   Y[y_offset + sum_i idx_i * y_strides[i]] = X[x_offset + sum_i idx_i * x_strides[i]]
 * for idx over `shape` (ndim <= 6, 4-byte elements of either dtype, offsets and
 * strides in elements).  x_strides may be negative (Slice with a negative
 * step); the whole view must lie inside both buffers. */
int wdh_strided_copy(wdh_buf X, int64_t x_offset, wdh_buf Y, int64_t y_offset,
                     int ndim, const int32_t *shape, const int64_t *x_strides,
                     const int64_t *y_strides);

#ifdef __cplusplus
}
#endif
#endif /* WEBDNN_HIP_H_ */
