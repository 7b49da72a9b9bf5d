/*
 * dr_hip.h -- the thin C-ABI device layer of the MI355X (gfx950) build of deepRacin.
 *
 * This is the layer the host graph code (the dR_* node implementations) calls instead of OpenCL.
 * It replaces the reference's OpenCL wrapper (src/dR_clwrap.c) and the clSetKernelArg /
 * clEnqueueNDRangeKernel sequences inside every node's compute() -- plain pointers and sizes only,
 * no C++ types, no torch types.  All kernels are hand-written HIP for gfx950 and compiled ahead of
 * time into libdeepracin.so; nothing is generated or compiled at run time.
 *
 * Conventions
 *   - every function returns 0 on success, a negative DRHIP_E* code on failure; a human readable
 *     message for the calling thread's last failure is available from drhip_last_error();
 *   - all device pointers are fp32 arrays; tensors are [C][H][W], x fastest (the reference's
 *     buffer layout, Kernels/dR_helper.cl:15-28);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); launches are
 *     asynchronous, only drhip_upload / drhip_download / drhip_stream_sync / drhip_event_elapsed_ms
 *     block;
 *   - launchers validate shapes on the host and refuse (DRHIP_EINVAL) instead of launching a grid
 *     that does not match what the kernel assumes.
 */
#ifndef DR_HIP_H
#define DR_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DRHIP_OK         0
#define DRHIP_EINVAL    -1   /* argument / shape rejected on the host, nothing launched */
#define DRHIP_EDEVICE   -2   /* a HIP runtime call failed */
#define DRHIP_ENODEVICE -3   /* no usable gfx950 device */

typedef struct drhip_device_info {
    char   name[256];
    char   arch[64];          /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int    device;            /* HIP ordinal */
    int    num_cu;            /* compute units */
    int    wavefront;         /* 64 on CDNA */
    int    lds_bytes;         /* max LDS per workgroup */
    int    clock_khz;
    size_t hbm_bytes;
    int    l2_bytes;
} drhip_device_info;

/* ---- runtime (replaces dR_clInit / dR_clCreateCLContext, reference src/dR_clwrap.c:4-235,592-872) */
int         drhip_init(int device, drhip_device_info* info /* may be NULL */);
const char* drhip_last_error(void);
int         drhip_device_count(void);          /* 0 when no device / no driver; never fails */

/* ---- streams and events (replace the in-order cl_command_queue, src/dR_clwrap.c:90, and the
 *      cl_event profiling of dR_finishCLKernel, src/dR_clwrap.c:955-1058) */
int drhip_stream_create(void** stream);
int drhip_stream_destroy(void* stream);
int drhip_stream_sync(void* stream);
int drhip_event_create(void** ev);
int drhip_event_destroy(void* ev);
int drhip_event_record(void* ev, void* stream);
int drhip_event_elapsed_ms(void* ev_start, void* ev_stop, float* ms);   /* waits for ev_stop */
/* Kernel execution times of the calling thread's launches: between drhip_timing_begin and
 * drhip_timing_end every kernel launch of this library carries its own start/stop event pair, so
 * ms[i] is the device time of launch i alone (what OpenCL's per-kernel profiling events gave the
 * reference, src/dR_clwrap.c:718-741).  drhip_timing_count = launches recorded so far;
 * drhip_timing_end waits for them and switches the recording off.  Not for use under capture. */
int drhip_timing_begin(void);
int drhip_timing_count(void);
int drhip_timing_end(float* ms, int capacity, int* count);
int drhip_stream_wait_event(void* stream, void* ev);      /* later work on `stream` starts after `ev`; joins a capture */
/* Measurement aid (no counterpart in the reference): the shader clock under a stream of fp32 MFMAs.  Two workgroups
 * per CU issue `iters` rounds of 8 independent v_mfma_f32_32x32x2_f32 per wave and read the shader-clock counter and
 * the constant 100 MHz counter around them; the kernel is launched `launches` times back to back (power management
 * reacts over milliseconds: a single short launch still sees idle clocks) and the last launch is read:
 * *mhz_median = median over its waves of the counters' ratio x 100 MHz, *microseconds (may be NULL) = median
 * duration of the measured stretch.  The data-sheet peak of the matrix cores
 * is quoted at 2400 MHz; utilisation figures against that peak are capped by this ratio.  Allocates and blocks. */
int drhip_mfma_clock_probe(int iters, int launches, float* mhz_median, float* microseconds, void* stream);

/* ---- launch graphs: record everything enqueued on `stream` between begin and end into an executable
 *      hipGraph and replay it with one call.  dR_apply uses it on request (DR_HIPGRAPH=1) to take the
 *      per-node launch cost (dozens of small kernels at batch 1) off the host.  capture_end returns DRHIP_EDEVICE and a NULL
 *      graph if something that cannot be captured (a blocking call, an allocation) happened in
 *      between; the stream is usable again afterwards. */
int drhip_graph_capture_begin(void* stream);
int drhip_graph_capture_end(void* stream, void** graph_exec);
int drhip_graph_launch(void* graph_exec, void* stream);
int drhip_graph_destroy(void* graph_exec);

/* ---- memory (replace dR_createFloatBuffer :886-899, dR_clMemoryBufferCleanup,
 *      dR_uploadArray :1079-1143 and dR_downloadArray :1145-1190; both copies block) */
int drhip_malloc(void** dptr, size_t bytes);
int drhip_free(void* dptr);
int drhip_upload(void* dst_dev, size_t dst_byte_offset, const void* src_host, size_t bytes, void* stream);
int drhip_download(void* dst_host, const void* src_dev, size_t src_byte_offset, size_t bytes, void* stream);
int drhip_fill_f32(float* dst, float value, size_t n, void* stream);
/* Staged transfers for the per-image copies of a serving loop (the feed of dR_feedData, the logits of
 * dR_downloadArray).  A staging object owns pinned host memory (hipHostMalloc): an upload area of
 * `upload_bytes` (two of them, used in turn) and a 64 KiB download area.  drhip_upload_staged copies the caller's (pageable) array
 * into an upload area and starts one transfer from there (up to 4 MiB: a kernel that reads the pinned
 * area, which starts sooner than the DMA engine; DR_UPLOAD_KERNEL=0 in the environment or larger arrays:
 * hipMemcpyAsync); it returns when the caller's array has been
 * read (the array may be reused), NOT when the data is on the device: the transfer is ordered on
 * `stream` before whatever is enqueued next.  An area is written again two uploads later; that the upload which
 * read it has finished follows from any staged download that completed on the same stream in between (the usual
 * feed / pass / download loop: nothing is recorded, nothing waited for); a caller that uploads again before any
 * download has completed gets an event recorded behind its upload, which the upload after the next waits for.
 * drhip_download_staged blocks like drhip_download; the data comes through the download area, stored
 * there by a small copy kernel (the area is mapped into the device's address space) that raises a flag
 * behind the data; the host watches the flag for up to DR_SPIN_US microseconds (default 1000; 0 = never)
 * before it waits for the stream the ordinary way - the flag is seen some 10 us before the stream's own
 * completion reaches the host.  One staging object serves one stream at a time.  Replace the blocking clEnqueueWriteBuffer / clEnqueueReadBuffer
 * of dR_uploadArray / dR_downloadArray (src/dR_clwrap.c:1079-1190) on the per-image path. */
int    drhip_staging_create(void** handle, size_t upload_bytes);
int    drhip_staging_destroy(void* handle);
size_t drhip_staging_upload_capacity(void* handle);
size_t drhip_staging_download_capacity(void* handle);
int    drhip_upload_staged(void* handle, void* dst_dev, size_t dst_byte_offset, const void* src_host, size_t bytes, void* stream);
int    drhip_download_staged(void* handle, void* dst_host, const void* src_dev, size_t src_byte_offset, size_t bytes, void* stream);

/* ---- convolution ------------------------------------------------------------------------------
 * Common meaning: in [I][H][W]; out [O][Ho][Wo] with Wo = W/strideX, Ho = H/strideY (floor);
 * zero padding of kw/2, kh/2; bias may be NULL; relu != 0 applies max(v,0) after the bias. */

/* Direct correlation, any odd kw x kh and any stride; w is [I][O][kh][kw] exactly as handed to
 * dR_Conv2d_setVariables.  out[o,y,x] = act(b[o] + sum_{c,j,i} in[c, y*sy+j-kh/2, x*sx+i-kw/2] * w[c][o][j][i]).
 * Replaces the per-layer generated kernel `conv2d<k>x<k>x<O>_<id>_...` and its launch
 * (reference src/dR_nodes_conv2d.c:364-420, 481-773); honours the stride as documented at
 * include/dR_nodes_conv2d.h:47-54. */
int drhip_conv2d_direct_f32(const float* in, const float* w, const float* bias, float* out,
                            int W, int H, int I, int O, int kw, int kh,
                            int strideX, int strideY, int relu, void* stream);

/* Direct 3x3 convolution (stride 1 or 2 in both directions, zero padding 1) as an implicit GEMM with
 * K = 9*I on the fp32 MFMA units, for layers with more than 4 input channels.  F is the filter bank in
 * the layout the kernel streams, produced once at prepare time from w [I][O][3][3]:
 * F[tap][c/8][o][8], tap = 3*j + i, input channels padded with zeros to a multiple of 8, output
 * channels to a multiple of 32, and channel c%8 stored at position (c&1)*4 + (c%8)/2 of its group of 8;
 * drhip_conv3x3_direct_filter_floats(I,O) floats.  `variant` (0 = let the launcher pick) = waves per
 * workgroup (1, 2, 4, 8: they deal the 8-channel stages round-robin, partial tiles added in wave
 * order) | 0x10 for 64 instead of 32 output channels per workgroup.  Same function as
 * drhip_conv2d_direct_f32 with kw = kh = 3.  Replaces the per-layer generated kernel
 * `conv2d3x3x<O>_<id>_...` and its launch (src/dR_nodes_conv2d.c:364-420, 481-773); the reference
 * re-lays nothing (it reads [I][O][3][3] through __constant or global memory).
 * W, H, I and O at most 65535 each (packed kernel arguments). */
size_t drhip_conv3x3_direct_filter_floats(int I, int O);
int drhip_conv3x3_direct_filter_layout_f32(const float* w /* [I][O][3][3] */, float* F, int I, int O, void* stream);
int drhip_conv3x3_direct_pick_variant(int Wo, int Ho, int I, int O);
int drhip_conv3x3_direct_mfma_f32(const float* in, const float* F, const float* bias, float* out,
                                  int W, int H, int I, int O, int stride, int relu, int variant, void* stream);

/* First layer (1 to 4 input channels, 3x3, any stride, zero padding, bias, optional ReLU) followed by
 * a 3x3 / stride-2 max pooling with the reference's pooling rules (out = ceil(in/2), samples outside
 * the map read 0.0): out[O][ceil(Ho/2)][ceil(Wo/2)], Wo = W/strideX, Ho = H/strideY.  The
 * convolution's own tensor is never written.  W, H and O at most 65535, strides at most 15 (packed kernel
 * arguments).  Replaces the generated conv kernel plus the generated
 * pooling kernel of such a pair (src/dR_nodes_conv2d.c:481-773, src/dR_nodes_pooling.c:277-401). */
int drhip_conv3x3_pool3s2_f32(const float* in, const float* w, const float* bias, float* out,
                              int W, int H, int I, int O, int strideX, int strideY, int relu, void* stream);

/* Winograd F(2x2,3x3) filter transform U = G g G^T for every (c,o).  Runs once per layer at
 * dR_prepare time.  U holds drhip_conv3x3_winograd_filter_floats(I,O) floats in the layout the MFMA
 * kernel streams: U[xi][c/8][o][8] with xi = 4*row+col, input channels padded with zeros to a
 * multiple of 8, and channel c%8 stored at position (c&1)*4 + (c%8)/2 of its group of 8.
 * Replaces the host loop of dR_conv2d_winograd_fillBuffers (src/dR_nodes_conv2d.c:1162-1240; the
 * reference stores [I][16][O]). */
size_t drhip_conv3x3_winograd_filter_floats(int I, int O);
int drhip_winograd_filter_transform_f32(const float* w /* [I][O][3][3] */, float* U, int I, int O, void* stream);

/* Fused Winograd F(2x2,3x3) convolution, stride 1, 3x3, SAME zero padding:
 * input transform B^T d B in registers, 16 transformed-domain [tiles x I].[I x O] products on the
 * fp32 MFMA units, output transform A^T m A + bias + ReLU, edge-guarded 2x2 stores.
 * `variant` is the configuration chosen by the scheduler: low 4 bits = output channels per
 * workgroup (1: 32, 2: 64, 3: 128), bits 4-7 = log2 of the number of input-channel splits, 0x100 =
 * blocks of 16 tiles (channels per workgroup then 16, 32, 64), 0x400 = eight waves per workgroup (two
 * wave sets that take alternate 8-channel stages; not with 32-tile blocks of 128 channels), 0x800 = joined
 * splits (below); 0 lets the launcher pick.  The input must be smaller than 2 GiB (32-bit byte offsets) and W, H, I and O at most 65535
 * each (the kernel carries them in 16-bit fields of its packed arguments; the graph layer sends larger layers to
 * drhip_conv2d_direct_f32).  A variant that splits the
 * input channels needs `workspace` of drhip_conv3x3_winograd_workspace_floats(...) floats (scratch,
 * no initialisation needed; two launches: partial tiles, then their sum in split order); otherwise
 * workspace may be NULL.  `relu` is a set of epilogue flags: DRHIP_EPILOGUE_RELU (1) and
 * DRHIP_EPILOGUE_MAXPOOL2 (2): `out` is then [O][H/2][W/2] and receives the 2x2 / stride-2 maximum
 * of every output tile instead of the tile (what a following max-pooling node with window and stride
 * (2,2,1) would compute, src/dR_nodes_pooling.c:277-401; W and H must be even).
 * Replaces kernel `conv2dwinograd2` and its launch
 * (Kernels/dR_winograd2.cl:23-254, src/dR_nodes_conv2d.c:1009-1132). */
#define DRHIP_EPILOGUE_RELU     1
#define DRHIP_EPILOGUE_MAXPOOL2 2
int drhip_conv3x3_winograd_f32(const float* in, const float* U, const float* bias, float* out,
                               int W, int H, int I, int O, int relu, int variant,
                               float* workspace, void* stream);
/* Variant id the gfx950 scheduler assigns to a layer of this shape; the counterpart of the
 * work-group search in dR_conv2d_winograd_schedule (src/dR_nodes_conv2d.c:809-1006). */
int drhip_conv3x3_winograd_pick_variant(int W, int H, int I, int O);
size_t drhip_conv3x3_winograd_workspace_floats(int W, int H, int I, int O, int variant);
/* Variants with bit 0x800 ("joined splits": 32-tile blocks, 2, 4, 8 or 16 equal input-channel splits, all workgroups
 * of the launch resident at once) add the splits' partial tiles up inside the one launch instead of in a second
 * kernel: every split finishes a slice of its panel and recognises a partial tile that has not arrived yet by the
 * marker value its workspace slot still holds.  The workspace of such a variant has to go through
 * drhip_conv3x3_winograd_workspace_prepare_f32 once (it fills in the marker, a signalling NaN that no sum can
 * produce); every launch leaves it prepared again, so it must not be shared with anything else and launches that use
 * it must not overlap.  drhip_conv3x3_winograd_f32 with variant 0 never picks a joined variant.  A partner that does
 * not deliver within the kernel's bounded wait (about 0.2 s: the device was shared so that the launch was not
 * resident as a whole) turns the affected outputs into NaN and is counted; drhip_conv3x3_winograd_join_timeouts
 * reads that count (a synchronous copy).  Environment DR_WINO_JOIN=0 keeps pick_variant from returning such variants.
 * Bit 0x1000 on top of 0x800 ("tiered", four waves, 32 or 64 channels per workgroup, split bits zero) lets the
 * launcher cut a layer whose blocks do not divide by the compute units into tiers: as many whole blocks per unit as fit,
 * then the rest halved, quartered ... over the input channels (joined as above) so that every unit gets the same
 * number of channel stages; the number of splits then differs per block and is not the caller's to choose.
 * Environment DR_WINO_TIERS=0 keeps pick_variant from returning it.
 * No counterpart in the reference: its kernel never splits the channel sum (Kernels/dR_winograd2.cl:176-189). */
int drhip_conv3x3_winograd_workspace_prepare_f32(float* workspace, size_t floats, void* stream);
int drhip_conv3x3_winograd_join_timeouts(unsigned* count);

/* 1x1 convolution as an fp32 MFMA GEMM out[O][P] = w[O x I] . in[I][P], P = H*W; w is the
 * original [I][O] array (no transpose needed).  Replaces kernel `conv2d1x1`, its launch and the
 * [I][O]->[O][I] re-layout (Kernels/dR_conv2d1x1.cl:4-53, src/dR_nodes_conv2d.c:1605-1716). */
int drhip_conv1x1_f32(const float* in, const float* w, const float* bias, float* out,
                      int P, int I, int O, int relu, int variant, void* stream);
/* 1x1 convolution followed by a global average pooling, without the [O][P] tensor in between:
 * partials[t*O + o] = sum over the pixels p of pixel tile t (32 pixels each) of act(b[o] + w . in[.][p]).
 * The pooled value of channel o is (sum_t partials[t*O + o]) / P: hand the partials to the consumer
 * as a drhip_deferred_vec {partials, NULL, drhip_conv1x1_poolsum_slices(P), O, 0, finished, P}.
 * No counterpart in the reference, which runs conv2d1x1 and the pooling kernel one after the other. */
int drhip_conv1x1_poolsum_slices(int P);
int drhip_conv1x1_poolsum_f32(const float* in, const float* w, const float* bias, float* partials,
                              int P, int I, int O, int relu, void* stream);
/* A 3x3 / stride-2 max pooling followed by a 1x1 convolution, without the pooled tensor in between:
 * in is the pooling's input [I][Hin][Win]; the convolution works on the pooled map of
 * ceil(Win/2) x ceil(Hin/2) pixels, whose samples it takes while loading (maximum over the window
 * anchored at (2x, 2y), samples outside the map count as 0.0); out is [O][ceil(Hin/2)][ceil(Win/2)].
 * Same values as drhip_pool_f32 followed by drhip_conv1x1_f32 up to the rounding of a channel sum that is
 * split over a different number of waves.  Replaces the generated
 * pooling kernel plus `conv2d1x1` of such a pair (src/dR_nodes_pooling.c:277-401,
 * Kernels/dR_conv2d1x1.cl:4-53). */
int drhip_conv1x1_pooled3s2_f32(const float* in, const float* w, const float* bias, float* out,
                                int Win, int Hin, int I, int O, int relu, void* stream);
/* Tile configuration for a 1x1 layer (replaces dR_conv2d_1x1_schedule, :1526-1602): waves per
 * output tile (1, 2, 4, 8 for 32x32 tiles; | 0x100 = 16x16 tiles, 1..16 waves, for small layers).
 * variant 0 in drhip_conv1x1_f32 = let the launcher pick. */
int drhip_conv1x1_pick_variant(int P, int I, int O);

/* ---- pooling ----------------------------------------------------------------------------------
 * out dims = ceil(in/stride) per axis; window anchored at (x*stx, y*sty, z*stz); samples outside
 * the input count as 0.0f; type 0 = max (start value -FLT_MAX), 1 = average (sum / (sx*sy*sz)).
 * `argmax_out` (may be NULL, max only) receives per output the flat input index of the first
 * maximum in z,y,x scan order, or -1 if the maximum is a padding zero.
 * Replaces the generated kernel `Pool<sx>x<sy>_<id>_nocopy{Max,Average}` and its launch
 * (reference src/dR_nodes_pooling.c:138-183, 277-401). */
int drhip_pool_f32(const float* in, float* out, int* argmax_out,
                   int W, int H, int C, int sx, int sy, int sz, int stx, int sty, int stz,
                   int type, void* stream);

/* ---- fully connected ---------------------------------------------------------------------------
 * y[n] = act(b[n] + sum_k x[k] * Wt[k][n]), Wt is [K][N] row-major (n fastest), x is the producer's
 * buffer read linearly.  The reference reads its [C][H][W] input in [H][W][C] order
 * (Kernels/dR_fcl.cl:78, Kernels/dR_helper.cl:131-142); the host folds that permutation into the
 * row order of Wt once at prepare time (drhip_fc_permute_rows_f32), so this kernel streams Wt
 * exactly once, contiguously.  `partials` is scratch of drhip_fc_scratch_floats(K,N) floats owned by
 * the caller (allocated at prepare time, no initialisation needed): the row range is split over
 * workgroups and a second small kernel sums the partial rows in fixed order (0 floats = the shape is
 * not split and partials may be NULL).  Replaces `matrixVectorMultFirst` + `matrixVectorMultSecond`
 * (Kernels/dR_fcl.cl:59-120, src/dR_nodes_fc.c:201-278). */
size_t drhip_fc_scratch_floats(int K, int N);
int drhip_fc_f32(const float* x, const float* Wt, const float* bias, float* y,
                 float* partials, int K, int N, int relu, void* stream);
/* Chains of GEMVs without the small kernels in between.  With `defer` != 0 a layer that is split
 * over row slices (drhip_fc_slices(K,N) > 1) stops after the partial sums: y is not written, and
 * the consumer is told where the sums are through a drhip_deferred_vec: element k of that vector is
 * act(bias[k] + sum_{s < slices} partials[s*n + k]), slices added in order - the value, bit for bit,
 * that the finishing kernel would have stored.  drhip_fc_ex_f32 and drhip_softmax_ex_f32 accept
 * such a vector as their input (`xdef` != NULL; x is then ignored) and, when `finished` is set,
 * store it there on the way.  No counterpart in the
 * reference, which always runs its second kernel (src/dR_nodes_fc.c:239-275). */
typedef struct drhip_deferred_vec {
    const float* partials;   /* [slices][n] */
    const float* bias;       /* [n] or NULL */
    int slices, n, relu;
    float* finished;         /* NULL, or [n]: the consumer also stores the finished vector here (for a
                                producer whose own output the caller wants to read) */
    float divisor;           /* 0, or the finished element is divided by this last (sums of a global
                                average pooling that its producer left as per-tile partial sums) */
} drhip_deferred_vec;
int drhip_fc_slices(int K, int N);
int drhip_fc_ex_f32(const float* x, const drhip_deferred_vec* xdef, const float* Wt, const float* bias, float* y,
                    float* partials, int K, int N, int relu, int defer, void* stream);
/* drhip_fc_f32 for callers that cannot allocate device memory and have none to lend (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same result, bit for bit, as drhip_fc_f32; the partial sums live in a 256 KiB array that
 * is part of the library's code object (one copy per GPU, held until the process ends, its address
 * looked up by drhip_init, which must have run for the current device).  The call allocates and
 * frees nothing.  Shapes whose partial sums exceed drhip_fc_noalloc_max_scratch_floats() floats
 * (drhip_fc_scratch_floats(K,N) tells) are refused with DRHIP_EINVAL; VGG16's three layers need
 * 65536, 65536 and 16000 (the limit is 65536; matrices of 33 000 to 65 000 columns need up to twice that).  All calls on one GPU share the array: calls that may overlap (different
 * streams, or graph branches) race on it; calls on one stream are safe.  Refused while
 * drhip_timing_begin is active. */
size_t drhip_fc_noalloc_max_scratch_floats(void);
int drhip_fc_noalloc_f32(const float* x, const float* Wt, const float* bias, float* y,
                         int K, int N, int relu, void* stream);
/* dst[k_chw][n] = src[k_hwc][n] with k_hwc = (y*W + x)*C + z for k_chw = (z*H + y)*W + x. */
int drhip_fc_permute_rows_f32(const float* src, float* dst, int W, int H, int C, int N, void* stream);

/* ---- normalization of a whole tensor (n elements) to a target mean and/or standard deviation:
 * type 0: y = x + (targetMean - mean); 1: y = x * (targetDev / dev); 2: both, dev = population
 * standard deviation about the mean.  Two (type 0) or three launches, no host round trip; `scratch`
 * = drhip_normalize_scratch_floats(n) floats, no initialisation needed.  x and y 16-byte aligned.
 * Replaces getAvg / getSumDev + blocking downloads + addScalar / mulScalar / addMulScalar
 * (src/dR_nodes_misc.c:1163-1446, Kernels/dR_helper.cl:315-471, Kernels/dR_math.cl:100-144). */
size_t drhip_normalize_scratch_floats(size_t n);
int drhip_normalize_f32(const float* x, float* y, size_t n, int type, float targetMean, float targetDev,
                        float* scratch, void* stream);

/* ---- softmax: y = exp(x - max x) / sum exp(x - max x) over n elements, one workgroup, wavefront
 * shuffles.  Replaces computeExp + host-side sum + mulScalar (src/dR_nodes_math.c:620-678,
 * Kernels/dR_math.cl:216-227,295-305). */
int drhip_softmax_f32(const float* x, float* y, int n, void* stream);
int drhip_softmax_ex_f32(const float* x, const drhip_deferred_vec* xdef, float* y, int n, void* stream);

/* ---- data movement nodes ------------------------------------------------------------------------
 * copy3d: dst[(z+dz0)][y+dy0][x+dx0] = src[(z+sz0)][y+sy0][x+sx0] for a (w,h,c) box; serves Concat
 * (generated kernel, src/dR_nodes_transform.c:468-553) and Slice (`extractSlice`,
 * Kernels/dR_transform.cl:5-24). */
int drhip_copy3d_f32(const float* src, int sW, int sH, int sx0, int sy0, int sz0,
                     float* dst, int dW, int dH, int dx0, int dy0, int dz0,
                     int w, int h, int c, void* stream);
/* y = f(x, s); op numbering = dR_ElemWise1OperationType: 0 x+s, 1 x-s, 2 x*s, 3 x/s, 4 log x, 5 exp x,
 * 6 sqrt x, 7 s, 8 pow(x,s)  (`addScalar` ... `powScalar`, Kernels/dR_math.cl:170-341) */
int drhip_scalar_op_f32(const float* x, float* y, size_t n, int op, float s, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DR_HIP_H */
