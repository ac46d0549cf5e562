/*
 * nncv_hip.h — C ABI of libnncv_hip.so, the MI355X (gfx950) implementation of nncv's
 * conv / GEMM / ResNet-18 hot path.
 *
 * Part 1 declares the symbols a program built against nncv already binds; replacing the object
 * file nncv-c produced (libres18.o) by this library needs no source change.
 * Part 2 declares device-resident forms of the same operations for callers that keep data in
 * HBM (benchmarks, serving loops); they have no counterpart in the reference, whose object only
 * knows host memory.
 *
 * All pointers are plain C; no C++ or framework types cross this boundary.
 */
#ifndef NNCV_HIP_H_
#define NNCV_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* MLIR strided memref descriptors, byte-identical to nncv::rt::MemRefDescriptor<T,N>
 * (include/libnncv/DataType.hpp:129-136): sizeof = 40 / 56 / 88 bytes for rank 1 / 2 / 4.
 * Element i.. is aligned[offset + sum_k i_k * strides[k]]; strides are in elements. */
typedef struct { void* allocated; void* aligned; intptr_t offset; intptr_t sizes[1]; intptr_t strides[1]; } nncv_memref1d;
typedef struct { void* allocated; void* aligned; intptr_t offset; intptr_t sizes[2]; intptr_t strides[2]; } nncv_memref2d;
typedef struct { void* allocated; void* aligned; intptr_t offset; intptr_t sizes[4]; intptr_t strides[4]; } nncv_memref4d;

/* ---------------------------------------------------------------------------------------------
 * Part 1 — the reference's ABI
 * ------------------------------------------------------------------------------------------- */

/* ResNet-18 forward, fp32, compiled with -split-params -wrap-c-interface.
 * Replaces the symbol declared in examples/Res18/main.cpp:18-23 and called at :96.
 *   dst    out: [N,1000]; the callee mallocs the buffer (64-byte aligned) and overwrites *dst,
 *          as MLIR's C interface does; the caller owns it afterwards.
 *   src    in : [N,3,H,W] NCHW host memory, any strides.
 *   params nncv_memref1d* over the flat model.bin blob (MemRefFlatArray::get(),
 *          src/libnncv/DataType.cpp:89-96), 11 699 112 fp32 elements in the canonical order
 *          (torchvision state_dict order without num_batches_tracked).
 * Errors (HIP failure, wrong parameter count, bad shape) print one "[ Erro ]" line to stderr and
 * abort(), the reference's convention (DnnModelLowering.cpp:222-230). */
void _mlir_ciface_forward(nncv_memref2d* dst, nncv_memref4d* src, void* params);

/* Same network from tests/Nets/Res18-half.mlir: every element is an IEEE half (uint16_t bits,
 * nncvFloat16 of DataType.hpp:127).  The reference object for it would carry the same symbol
 * name as the fp32 one; one library cannot export both, hence the suffix. fp32 accumulation. */
void _mlir_ciface_forward_f16(nncv_memref2d* dst, nncv_memref4d* src, void* params);

/* linalg.matmul: res = c + a.b, fp32 row-major (tests/MatMulOptimization/MatMulDeafult.mlir:6-9).
 * The product is accumulated into c's buffer in place and *res aliases it. */
void _mlir_ciface_matmul(nncv_memref2d* res, nncv_memref2d* a, nncv_memref2d* b, nncv_memref2d* c);

/* linalg.conv_2d_nchw_fchw: res = out + conv(in, filter), fp32, `in` already padded
 * (tests/ConvOptimization/Conv2dNchwFchwManually.mlir:7-13).  The stride is a compile-time
 * attribute in the reference; here it is recovered from the shapes:
 * stride = (H - R) / (OH - 1) (1 when OH == 1), and the shapes must then be consistent.
 * Accumulates into out's buffer in place; *res aliases it. */
void _mlir_ciface_batch_nchw_conv(nncv_memref4d* res, nncv_memref4d* in, nncv_memref4d* filter, nncv_memref4d* out);

/* ---------------------------------------------------------------------------------------------
 * Part 2 — device-resident forms (no counterpart in the reference)
 * Return 0 on success, non-zero on error; nncv_hip_last_error() then describes it.
 * dtype: 1 = fp32, 2 = fp16 (numbering of nncv::rt::dataType, DataType.hpp:118-124).
 * `stream` is a hipStream_t passed as void* (NULL = the library's own stream, after which the
 * call synchronises; with a caller stream the call only enqueues).
 * ------------------------------------------------------------------------------------------- */
int nncv_hip_init(int device);            /* optional; device < 0 keeps the current device */
const char* nncv_hip_last_error(void);
const char* nncv_hip_device_arch(void);   /* e.g. "gfx950:sramecc+:xnack-" */

/* Per-kernel timing with HIP events on the launch stream. While enabled every kernel launch is
 * bracketed by two events; nncv_hip_profile_report waits for them, writes a JSON object
 * {tag: {"launches", "ms", "flops", "bytes"}} (algorithmic flops / bytes as declared by each
 * launcher) into buf (at most cap bytes, NUL terminated), clears the records and returns the size
 * the full text needs. */
void nncv_hip_profile_enable(int on);
size_t nncv_hip_profile_report(char* buf, size_t cap);

/* conv algorithms for 3x3 stride-1 layers */
#define NNCV_HIP_ALGO_AUTO 0
#define NNCV_HIP_ALGO_WINOGRAD 1 /* F(4x4,3x3): input/filter/output transforms + 36 batched GEMMs */
#define NNCV_HIP_ALGO_IGEMM 2    /* implicit GEMM on MFMA */

typedef struct nncv_hip_model nncv_hip_model;
/* params: HOST pointer to the flat blob (n_elems elements of `dtype`). Uploads, folds BN, re-lays
 * and transforms the filters once. */
nncv_hip_model* nncv_hip_resnet18_create(const void* params, int64_t n_elems, int dtype, int algo3x3);
/* The same, for a caller that keeps `passes_in_flight` forward passes in flight at once (this handle and its clones, each
 * on a stream of its own; nncv_hip_pick_streams finds streams that overlap).  The value belongs to the handle: from 3 up
 * its launches take the shapes that measured faster when launches of several passes share the chip (fewer, larger
 * workgroups in the fp16 3x3 kernel; no lingering of tensors in the workspace; average pool and FC as two small
 * launches): ResNet-18 fp16 at batch 32 with four passes in flight 0.159 against 0.168 ms per pass, but 0.275 against
 * 0.256 ms with one pass at a time.  Results are the same tensors either way, and handles with different values work
 * side by side in one process.  0 = follow the process-wide default (nncv_hip_set_overlap_hint).  No counterpart in the
 * reference, whose compiled forward is one synchronous CPU call (examples/Res18/main.cpp:95-99). */
nncv_hip_model* nncv_hip_resnet18_create_ex(const void* params, int64_t n_elems, int dtype, int algo3x3, int passes_in_flight);
/* the value the handle plans with (its own, or the process-wide default); -1 for a null handle */
int nncv_hip_resnet18_passes_in_flight(const nncv_hip_model* m);
/* `want` (1..8) HIP streams for keeping several passes in flight, written to streams[0..want) as hipStream_t.  Streams
 * of one process share a few hardware queues, and queues share the command processor's four pipes; work on two streams
 * overlaps only when they landed on different pipes, which cannot be asked, so the library measures it once per process
 * (about 40 ms: chains of short one-wave kernels on eight candidate streams, pairwise) and hands out the streams that ran
 * side by side first.  *overlapping (may be NULL) = how many of the returned streams overlap pairwise; the rest fill the
 * list up.  More hardware queues (GPU_MAX_HW_QUEUES=8 in the environment before the process first touches HIP) make
 * four overlapping streams more likely.  Call it while the device is otherwise idle (other work disturbs the timing).
 * The streams have the default priority, belong to the library and live until the process ends.  No counterpart in
 * the reference. */
int nncv_hip_pick_streams(int want, void** streams, int* overlapping);
void nncv_hip_resnet18_destroy(nncv_hip_model* m);
/* A second handle on the SAME device weights (fp16 models only; an fp32 model keeps the tickets of its K-split launches
 * with its layers, which two passes at once would share): its own workspace, so its passes overlap with those of
 * `m` and of other clones on other streams like those of separately created models do, without a second copy of the
 * 23 MB of filters in memory and in the caches (four passes in flight: 0.160 against 0.163 ms per pass).  The weights
 * live until the last handle on them is destroyed.  NULL on error.  No counterpart in the reference, whose compiled
 * forward is stateless (examples/Res18/main.cpp:95-99). */
nncv_hip_model* nncv_hip_resnet18_clone(nncv_hip_model* m);  /* inherits passes_in_flight */
/* src: DEVICE NCHW [N,3,H,W] of the model's dtype; logits: DEVICE [N,1000] fp32.  `stream`: the caller's HIP stream
 * (the call only enqueues), or NULL for the library's own stream (the call then returns when the pass is done).
 * A handle owns its workspace: passes of different handles on different streams run concurrently (two passes in
 * flight fill each other's launch gaps -- the way to the highest throughput); calls on one handle are ordered one
 * after the other, also across streams. */
int nncv_hip_resnet18_forward(nncv_hip_model* m, const void* src, int N, int H, int W, float* logits, void* stream);

/* Same, and also copies the NHWC activation after `stage` (0: after the max-pool, 1..4: after
 * layer1..layer4) of the model's dtype to DEVICE `tap` — for layer-by-layer parity checks. */
int nncv_hip_resnet18_forward_tap(nncv_hip_model* m, const void* src, int N, int H, int W, float* logits, int stage,
                                  void* tap, void* stream);

typedef struct nncv_hip_conv nncv_hip_conv;
/* One fused conv + BN + (residual) + activation layer. weights: HOST FCHW of `dtype`;
 * bn: HOST gamma, beta, mean, var of `dtype`, each [F], or all NULL; relu: 0 none, 1 ReLU, or any
 * other NNCV_HIP_ACT_* code (those run on the implicit-GEMM kernels only). */
nncv_hip_conv* nncv_hip_conv_create(int dtype, const void* weights, int F, int C, int R, int S, int stride, int pad,
                                    const void* gamma, const void* beta, const void* mean, const void* var, int relu,
                                    int algo);
void nncv_hip_conv_destroy(nncv_hip_conv* c);
int nncv_hip_conv_algo(const nncv_hip_conv* c);
/* layout: 0 = NCHW, 1 = NHWC for in, out and residual alike (DEVICE pointers of the layer's dtype);
 * in is [N,C,H,W] UNPADDED, out [N,F,OH,OW]; residual may be NULL. NHWC is the native layout. */
int nncv_hip_conv_forward(nncv_hip_conv* c, const void* in, int N, int H, int W, int layout, const void* residual,
                          void* out, void* stream);
/* The same as nncv_hip_conv_forward with layout = 1 (NHWC), for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The
 * workspace the layer's kernels need (the partial sums and ticket counters of the K split of fp32 3x3 layers) is a
 * device array of the library, 4 MiB + 1 KiB on every GPU it runs on, held until the process ends; the call allocates
 * and frees nothing.  A layer/shape whose workspace is larger fails with an error that says so.  All calls on one GPU
 * share the array.  Outside a capture the library orders them itself: a call on another stream than the previous one
 * first waits for the event that call left behind.  On a stream that is being captured it neither waits nor records
 * (either would end the capture): the recorded launches run when the caller's graph does, and keeping two such graphs,
 * or a graph and eager calls, from overlapping in time on one GPU is then the caller's business -- they would race. */
int nncv_hip_conv_forward_noalloc(nncv_hip_conv* c, const void* in, int N, int H, int W, const void* residual, void* out,
                                  void* stream);
/* Measurement helper: `reps` NHWC launches of the layer back to back on `stream` between one pair
 * of HIP events (after 5 untimed ones); *avg_us = elapsed / reps. Includes the gap between
 * consecutive dispatches, so it reads slightly above a profiler's per-kernel time. */
int nncv_hip_conv_time(nncv_hip_conv* c, const void* in, int N, int H, int W, const void* residual, void* out, int reps,
                       void* stream, float* avg_us);
/* The handle-less entry points (_mlir_ciface_forward and its fp16 / MobileNetV3 forms) keep the device copy of a
 * parameter blob between calls, keyed by the blob's host address, length and type, and notice new contents at the same
 * address through a fingerprint of 4096 evenly spaced samples (hashing all 47 MB on every call would cost more than the
 * forward pass).  A caller that rewrites parameters in place calls this afterwards: the device copies made from
 * `params` (all of them when `params` is NULL) are dropped and rebuilt on the next call.  Returns 0.  No counterpart
 * in the reference, whose compiled forward re-reads the blob on every call (examples/Res18/main.cpp:95-99). */
int nncv_hip_params_invalidate(const void* params);
/* The process-wide DEFAULT of passes_in_flight (see nncv_hip_resnet18_create_ex): what handles created without a value
 * of their own, the operator-list executor and the single-layer entry points plan with (1 = one pass after the other,
 * the initial value unless NNCV_HIP_OVERLAP says otherwise).  Handles that carry their own value are not affected.  A
 * change waits for the device and drops every captured graph, so call it between phases, not per pass.  Returns 0.
 * No counterpart in the reference. */
int nncv_hip_set_overlap_hint(int passes);
/* Diagnostic, host arithmetic only (works without a GPU): the tile plan of the 3x3 LDS-patch kernel for
 * N x OH x OW output pixels at `stride` (1 | 2), F filters and `slabs` 128-byte channel slabs.
 * plan[8] = {WS (64-slot groups per workgroup), TN images, TH rows, TW columns per tile, NTX column tiles per
 * row band, log2 of the loader's row walk, LDS cells available, pixels the loader can walk}.  Returns 0, or 1 when
 * no plan exists. No counterpart in the reference: it lets the CPU test suite check the planner's invariants
 * (a plan that overflows LDS or the loader would fault on the device). */
int nncv_hip_conv3x3_patch_plan(int stride, int N, int OH, int OW, int F, int slabs, int* plan);
/* Diagnostic, host arithmetic only: the launch plan of the fp16 3x3 stride-1 stream kernel for N x H x W pixels, C
 * channels and F filters.  plan[14] = {TH virtual rows per tile, S virtual rows per image, top (1: the images are one
 * zero row apart), aligned (1: tiles never leave their image), tiles, NSEG seven-cell segments per patch row, PG pixel
 * groups, WF filter groups, WK K groups of a workgroup, filter blocks, workgroups per filter block (= the tile step of a
 * workgroup), row segments one patch buffer holds, spare bytes behind the segments of a patch row (they bring the row
 * pitch to 9 W sixteen-byte units mod 16, which keeps the pixel reads free of bank conflicts; 0: plain segment rows),
 * bytes of one patch buffer}.  Returns 0, or 1 when the kernel does not take the shape.
 * No counterpart in the reference: it lets the CPU test suite check that a plan never outgrows the kernel's LDS. */
int nncv_hip_conv3x3_stream_plan(int N, int H, int W, int C, int F, int* plan);

/* The reference driver's image preparation and top-1 scan on the device
 * (examples/Res18/main.cpp:38-77 and :103-111).
 * preprocess: hwc_u8 is a DEVICE [N,H,W,channels] 8-bit image (channels 3 or 4, the first three
 * used); nchw_out receives [N,3,H,W] of `dtype` with x = ((u8 / 255.f) - mean[c]) / std[c], mean =
 * {0.485, 0.456, 0.406}, std = {0.229, 0.224, 0.225}, fp32 arithmetic in that order.
 * argmax: top1[n] = the first index of the largest of logits[n][0..F) that exceeds -100 (0 if none;
 * NaNs never win) -- the driver's loop. classify_u8 = preprocess + forward + argmax in one call;
 * logits [N,1000] fp32 and top1 [N] are DEVICE buffers. */
int nncv_hip_preprocess_u8(const void* hwc_u8, int N, int H, int W, int channels, int dtype, void* nchw_out, void* stream);
int nncv_hip_argmax(const float* logits, int N, int F, int* top1, void* stream);
int nncv_hip_resnet18_classify_u8(nncv_hip_model* m, const void* hwc_u8, int N, int H, int W, int channels, float* logits,
                                  int* top1, void* stream);

/* Activation arena planner: "greedy by size" offset calculation of arXiv 2001.03288 sec. 5.2, the
 * algorithm of the reference's MemSolver (src/nncv/compiler/Optimizer/MemSolver.cpp:15-47; known
 * answer tests/MemSolver/test.cpp:17-37 = 124). Tensor i is live during operators
 * first_op[i]..last_op[i] (inclusive) and needs bytes[i]; offsets[i] receives its place in one
 * allocation whose size is returned (~0 on error). Host-only, needs no device. The ResNet-18
 * workspace of this library is laid out with it. */
unsigned long long nncv_hip_plan_arena(int n, const int* first_op, const int* last_op, const unsigned long long* bytes,
                                       unsigned long long align, unsigned long long* offsets);

/* C += A.B, fp32 row-major, DEVICE pointers, any M, N, K >= 1 (the device form of _mlir_ciface_matmul;
 * tests/MatMulOptimization/MatMulDeafult.mlir:11-21). */
int nncv_hip_matmul_f32(const float* A, const float* B, float* C, int M, int N, int K, void* stream);
/* Measurement helper, like nncv_hip_conv_time: `reps` launches of C += A.B back to back on `stream` between one pair
 * of HIP events (after 5 untimed ones); *avg_us = elapsed / reps.  C keeps accumulating. */
int nncv_hip_matmul_time(const float* A, const float* B, float* C, int M, int N, int K, int reps, void* stream, float* avg_us);

/* Winograd F(4x4,3x3) stages on DEVICE buffers (layouts: U[36][F][C], V[36][tiles][C], M[36][tiles][F],
 * tiles = N*ceil(OH/4)*ceil(OW/4)); exposed so each stage can be checked and profiled alone. */
int nncv_hip_wino43_filter(int dtype, const void* w_fchw, void* U, int F, int C, void* stream);
int nncv_hip_wino43_input(int dtype, const void* in, int layout, void* V, int N, int C, int H, int W, int pad, void* stream);
int nncv_hip_wino43_gemm(int dtype, const void* V, const void* U, void* M, int64_t tiles, int C, int F, void* stream);
int nncv_hip_wino43_output(int dtype, const void* M, void* out, int layout, int N, int F, int OH, int OW,
                           const float* scale, const float* shift, const void* residual, int relu, void* stream);

/* pooling on DEVICE NHWC tensors */
int nncv_hip_maxpool3x3s2(int dtype, const void* in, void* out, int N, int H, int W, int C, void* stream);
int nncv_hip_global_avgpool(int dtype, const void* in, void* out, int N, int H, int W, int C, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Network graphs: the other fixtures of tests/Nets (MobileNetV3.mlir: depthwise convolution,
 * hard-swish, squeeze-excitation; Yolov5s.mlir: SiLU, concatenation, up-sampling, 5x5 max-pool)
 * as a list of fused operators over numbered tensors. Tensor 0 is the network input; every other
 * tensor is the `out` of exactly one operator and is read only by later ones; the `out` of the
 * last operator is the network output. No counterpart in the reference (its compiler bakes the
 * graph into code); the operator vocabulary is the fixtures'.
 * ------------------------------------------------------------------------------------------- */
#define NNCV_HIP_OP_CONV 1        /* conv_2d_nchw_fchw (+bias) (+BatchNorm) (+ in[1] residual) + act; a Linear layer is K = 1 */
#define NNCV_HIP_OP_DWCONV 2      /* depthwise_conv_2d_nchw_chw (+bias) (+BatchNorm) + act; K = 3 or 5 */
#define NNCV_HIP_OP_MAXPOOL 3     /* pooling_nchw_max K x K, -inf halo of `pad` */
#define NNCV_HIP_OP_GAVGPOOL 4    /* pooling_nchw_sum over the whole image / (H*W) -> [N,C,1,1] */
#define NNCV_HIP_OP_SCALE 5       /* out = in[0] * in[1], in[1] of shape [N,C,1,1] */
#define NNCV_HIP_OP_ADD 6         /* out = act(in[0] + in[1]) */
#define NNCV_HIP_OP_ACT 7         /* out = act(in[0]) */
#define NNCV_HIP_OP_CONCAT 8      /* out = concat over channels of in[0..3] (unused = -1) */
#define NNCV_HIP_OP_UPSAMPLE2X 9  /* nearest-neighbour, H and W doubled */
/* YOLOv5 Detect decode (tests/Nets/Yolov5s.mlir:1348-1448), only as the LAST operator: in[0..2] are the
 * head tensors of up to three levels, each with K * F channels (K anchors per level, F = 5 + classes
 * values per anchor). w: anchors [levels,K,2] in units of the level's stride, bias: strides [levels].
 * s = sigmoid(head); xy = (2 s + grid - 0.5) * stride; wh = (2 s)^2 * anchor * stride; the rest is s.
 * Network output: [N, sum_l K*H_l*W_l, F] fp32, boxes ordered (level, anchor, y, x); reported by
 * nncv_hip_graph_output_shape as channels = boxes, height = F, width = 1. */
#define NNCV_HIP_OP_YOLO_DETECT 10

#define NNCV_HIP_ACT_NONE 0
#define NNCV_HIP_ACT_RELU 1         /* select(x ugt 0, x, 0) */
#define NNCV_HIP_ACT_HARDSWISH 2    /* (min(relu(x + 3), 6) / 6) * x */
#define NNCV_HIP_ACT_HARDSIGMOID 3  /* max(0, min(1, (x + 3) / 6)) */
#define NNCV_HIP_ACT_SILU 4         /* x * (1 / (1 + exp(-x))) */
#define NNCV_HIP_ACT_SIGMOID 5

typedef struct nncv_hip_graph_op {
  int32_t kind;
  int32_t in[4];   /* tensor ids, unused = -1 */
  int32_t out;     /* tensor id */
  int32_t F;       /* CONV: filters */
  int32_t K, stride, pad;
  int32_t act;
  float eps;       /* BatchNorm epsilon (used when gamma >= 0) */
  /* element offsets into the parameter blob, -1 = absent.  w: [F,C,K,K] (DWCONV: [C,1,K,K]);
   * bias, gamma, beta, mean, var: [F].  y = BN(conv + bias) */
  int64_t w, bias, gamma, beta, mean, var;
} nncv_hip_graph_op;

typedef struct nncv_hip_graph nncv_hip_graph;
/* params: HOST pointer to n_elems elements of `dtype`. Channel counts that are not multiples of 8
 * (fp16) / 4 (fp32) are allowed for the network input and for convolution outputs that feed only
 * convolutions, YOLO_DETECT or the network output (they are stored padded). Returns NULL on error
 * (nncv_hip_last_error). */
nncv_hip_graph* nncv_hip_graph_create(const nncv_hip_graph_op* ops, int n_ops, int in_channels, const void* params,
                                      int64_t n_elems, int dtype);
void nncv_hip_graph_destroy(nncv_hip_graph* g);
/* shape[3] = channels, height, width of the network output for an H x W input */
int nncv_hip_graph_output_shape(const nncv_hip_graph* g, int H, int W, int* shape);
/* src: DEVICE NCHW [N,in_channels,H,W] of the graph's dtype; out: DEVICE NCHW fp32 of the output
 * shape, out_elems = N*C*OH*OW (checked). */
int nncv_hip_graph_forward(nncv_hip_graph* g, const void* src, int N, int H, int W, float* out, int64_t out_elems,
                           void* stream);
/* The workspace plan nncv_hip_graph_forward would use for an [N,in_channels,H,W] input, computed on the
 * HOST (no device is touched, no parameters are needed): the planner is the greedy-by-size offset
 * calculation of the reference's MemSolver (src/nncv/compiler/Utils/MemSolver.cpp:15-47) over tensor
 * lifetimes that follow the launches actually issued (merged operators write at the merged launch).
 * tensor_info[4*t .. 4*t+3] = {id of the tensor whose memory block t lives in (itself unless it is a
 * slice of a concatenated tensor), byte offset of t, bytes of that block, channel offset of t in it};
 * launch_dst[i] = tensor the launch of operator i writes, -1 if the operator is merged into another
 * launch or writes the caller's buffer. Refuses (-1) a plan in which a launch would write over memory
 * it reads. Returns the workspace bytes. */
int64_t nncv_hip_graph_plan(const nncv_hip_graph_op* ops, int n_ops, int in_channels, int dtype, int N, int H, int W,
                            int64_t* tensor_info, int tensor_cap, int32_t* launch_dst);
/* The operator list of torchvision's MobileNetV3-small as exported in tests/Nets/MobileNetV3.mlir
 * (parameters in state_dict order without num_batches_tracked). Writes at most `cap` operators,
 * returns their number; *n_elems receives the parameter count. _mlir_ciface_forward serves this
 * network too when handed a params memref of that many elements. */
int nncv_hip_mobilenetv3_small_ops(nncv_hip_graph_op* ops, int cap, int64_t* n_elems);

/* Single operators of the list above on DEVICE NHWC tensors of `dtype` (for parity checks).
 * dwconv: w is DEVICE [C,1,K,K]; scale / shift DEVICE fp32 [C] or NULL. */
int nncv_hip_dwconv(int dtype, const void* in, const void* w, const float* scale, const float* shift, void* out, int N, int H,
                    int W, int C, int K, int stride, int pad, int act, void* stream);
int nncv_hip_scale_channels(int dtype, const void* x, const void* gate, void* out, int N, int HW, int C, void* stream);
int nncv_hip_eltwise(int dtype, const void* a, const void* b, void* out, int64_t n, int act, void* stream);
int nncv_hip_concat_slice(int dtype, const void* x, void* out, int64_t P, int C, int ldo, int c0, void* stream);
int nncv_hip_upsample2x(int dtype, const void* x, void* out, int N, int H, int W, int C, int ldo, int c0, void* stream);
int nncv_hip_maxpool(int dtype, const void* in, void* out, int N, int H, int W, int C, int K, int stride, int pad, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NNCV_HIP_H_ */
