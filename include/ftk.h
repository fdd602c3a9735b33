/*
 * ftk.h -- C ABI of libftkernels.so: MI355X (gfx950) kernels for the
 * FractalTensor hot path (fused LSTM cell scan, stacked / dilated LSTM,
 * back-to-back fp16 GEMM, flash attention with online softmax).
 *
 * Conventions (all entry points):
 *   - plain C, no C++/torch types; every pointer argument is a DEVICE pointer
 *     owned by the caller unless its comment says "host";
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     calls are stream-ordered and asynchronous, nothing synchronises;
 *   - the return value is 0 on success and a negative FTK_ERR_* code on
 *     failure; ftk_last_error() returns a thread-local description of the
 *     last failure.  Nothing exits, aborts or throws;
 *   - no entry point allocates device memory: kernels that need scratch take
 *     a caller-provided workspace whose size the matching
 *     *_workspace_bytes() function reports;
 *   - matrices are dense row-major with the last index contiguous, and start
 *     at a 16-byte boundary (every device allocator's do); the entry points
 *     that say so return FTK_ERR_INVALID_ARGUMENT for one that does not.
 *
 * The reference (microsoft/FractalTensor) has no C ABI of its own: its
 * kernels are compile-time-shaped C++ functors called from gtest/benchmark
 * binaries, and its Python frontend never reaches them.  Each declaration
 * below names the reference functor or Python function it stands in for.
 */
#ifndef FTK_H_
#define FTK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FTK_OK 0
#define FTK_ERR_INVALID_ARGUMENT (-1) /* null pointer, non-positive size          */
#define FTK_ERR_UNSUPPORTED_SHAPE (-2) /* shape outside what the kernels tile for */
#define FTK_ERR_WORKSPACE (-3)        /* workspace missing or too small           */
#define FTK_ERR_LAUNCH (-4)           /* HIP reported an error at launch          */
#define FTK_ERR_DEVICE (-5)           /* device query failed / not a gfx950 part  */
#define FTK_ERR_TIMEOUT (-6)          /* a persistent launch gave up waiting: see ftk_stacked_lstm_status() */

typedef void* ftk_stream_t;

typedef struct ftk_device_info {
  int compute_units;       /* multiProcessorCount                               */
  int lds_bytes_per_block; /* sharedMemPerBlock opt-in maximum                  */
  int clock_khz;           /* engine clock                                      */
  int wavefront_size;      /* 64 on CDNA                                        */
  int persistent_slots;    /* co-resident 256-thread, full-register workgroups  */
  char arch[32];           /* gcnArchName, e.g. "gfx950:sramecc+:xnack-"        */
} ftk_device_info;

/* Library version, major*10000 + minor*100 + patch. */
int ftk_version(void);

/* Thread-local text for the most recent non-zero return on this thread. */
const char* ftk_last_error(void);

/* Properties of the current HIP device.
 * Stands in for GPUContext / GetGPUComputeCapability
 * (kaleido/core/device/gpu_context.h:11-64, kaleido/core/device/cuda_info.h). */
int ftk_device_info_query(ftk_device_info* out);

/* ---------------------------------------------------------------- LSTM -- */

/*
 * One batched LSTM cell, gate GEMM and state update fused in one launch:
 *   g = [x, h_prev] @ WU + bias,  column blocks of g: i | f | o | c~
 *   c = sigmoid(f)*c_prev + sigmoid(i)*tanh(c~);  h = sigmoid(o)*tanh(c)
 * x [B,I], h_prev/c_prev [B,H] (both NULL = zero state), WU [(I+H),4H],
 * bias [4H] or NULL, outputs h/c [B,H].  fp32.  Needs I%32==0, H%32==0.
 * Replaces CuteLSTMCell::operator() (kaleido/core/device/kernels/lstm.h:253-348:
 * KeCuteLSTMGate lstm_kernels.h:25-126 + KeLSTMElementWise lstm/inner.h:595-662)
 * and the Python lstm_cell (examples/stacked_rnn/stacked_rnn.py:23-36).
 */
int ftk_lstm_cell_f32(const float* x, const float* h_prev, const float* c_prev,
                      const float* WU, const float* bias, float* h, float* c,
                      int B, int I, int H, ftk_stream_t stream);

/*
 * The same cell with fp16 storage: x, h_prev, c_prev, WU, h, c fp16, bias fp32
 * or NULL; gate sums and the state update in fp32, h and c rounded to fp16 when
 * written.  Needs I%32==0, H%32==0.  The weights are streamed through LDS, so
 * any hidden size runs; a workgroup takes 256 batch rows, which at B <= 256
 * fetches every weight once.  The element types of CuteLSTMCell as the
 * reference instantiates it (cutlass::half_t, kaleido/core/device/kernels/lstm.h:253-348;
 * fp32 accumulators, lstm_kernels.h:25-126).
 */
int ftk_lstm_cell_f16(const void* x, const void* h_prev, const void* c_prev,
                      const void* WU, const float* bias, void* h, void* c,
                      int B, int I, int H, ftk_stream_t stream);

/*
 * One LSTM layer over T steps from a given initial state: step t is the cell
 * above on xs[t] and the state of step t-1 (h0, c0 for t = 0; both NULL = zero
 * state).  xs [T,B,I], WU [(I+H),4H], bias [4H] or NULL, h0/c0 [B,H],
 * outputs hs/cs [T,B,H].  One fused-cell launch per step on the stream.
 * _f32: all fp32; _f16: xs, WU, h0, c0, hs, cs fp16, bias fp32.
 * Needs I%32==0, H%32==0.  Replaces CuteLSTMLayer::operator()(w, xs, u, c_init,
 * h_init, csss, hsss, seq_length) (kaleido/core/device/kernels/lstm.h:479-602)
 * and the Python lstm_layer (examples/stacked_rnn/stacked_rnn.py:54-65).
 */
int ftk_lstm_layer_f32(const float* xs, const float* WU, const float* bias,
                       const float* h0, const float* c0, float* hs, float* cs,
                       int T, int B, int I, int H, ftk_stream_t stream);
int ftk_lstm_layer_f16(const void* xs, const void* WU, const float* bias,
                       const void* h0, const void* c0, void* hs, void* cs,
                       int T, int B, int I, int H, ftk_stream_t stream);

/*
 * The state-update half alone, for the unfused baseline: gates [B,4H] already
 * holds x@W + h@U (pre-activation, blocks i|f|o|c~); bias [4H] or NULL;
 * c_prev [B,H] or NULL.  Replaces ElementwiseLstmAct
 * (kaleido/core/device/kernels/elementwise.h:141-155) as used by
 * benchmarks/rnn/fractaltensor/utils.h:439-495.
 */
int ftk_lstm_elementwise_f32(const float* gates, const float* bias,
                             const float* c_prev, float* h, float* c, int B,
                             int H, ftk_stream_t stream);

/* Bytes of workspace ftk_stacked_lstm_f32 / ftk_dilated_lstm_f32 need. */
size_t ftk_stacked_lstm_workspace_bytes(int L, int T, int B, int H);

/*
 * L stacked LSTM layers over T steps; layer l reads layer l-1's hidden
 * sequence; zero initial state.  xs [T,B,H], WU [L,2H,4H], bias [L,4H] or
 * NULL, outputs hsss/csss [L,T,B,H] (every layer's h and c at every step).
 * H%32==0.  At H = 256 one persistent launch walks the (layer,time) wavefront
 * with each layer's weights held in registers.  Other hidden sizes do not fit
 * on chip and run as one fused-cell launch per wavefront diagonal with the
 * weights streamed: in the default product mode (see ftk_lstm_set_products)
 * through the fp16-MFMA kernel on operands split into two fp16 planes, for
 * which the workspace holds the planes of xs and of every h, the column
 * scales and a re-laid copy of the split weights (about 1.5x the bytes of WU
 * plus those of hsss; ftk_stacked_lstm_workspace_bytes says how much); with a
 * smaller workspace or in the fp32-product mode through the fp32-MFMA cell
 * kernel of ftk_lstm_cell_f32, which needs none.
 * Replaces StackedLstmRegion1/2/3
 * (kaleido/core/device/kernels/lstm/stacked_lstm/region1.h:11-43,
 * region2.h:15-70, region3.h:18-140) and the Python stacked_lstm
 * (examples/stacked_rnn/stacked_rnn.py:54-79).
 */
int ftk_stacked_lstm_f32(const float* xs, const float* WU, const float* bias,
                         float* hsss, float* csss, int L, int T, int B, int H,
                         void* workspace, size_t workspace_bytes,
                         ftk_stream_t stream);

/*
 * Same with a per-layer dilation: layer l takes its state from step
 * t - dilations[l] (zero state for t < dilations[l]).  `dilations` is a HOST
 * array of L positive ints.  Replaces DilatedLstmRegion1/2
 * (kaleido/core/device/kernels/lstm/dilated_lstm/region1.h:13-29,
 * region2.h:12-82) and dilated_layer/model of
 * examples/dilated_rnn/dilated_rnn.py:16-41.
 */
int ftk_dilated_lstm_f32(const float* xs, const float* WU, const float* bias,
                         const int* dilations, float* hsss, float* csss, int L,
                         int T, int B, int H, void* workspace,
                         size_t workspace_bytes, ftk_stream_t stream);

/*
 * The same for a ragged batch in the time-major layout: rows sorted by
 * decreasing length, active_rows[t] (a HOST array of T ints, non-increasing,
 * each in [0,B]) = how many leading rows are still running at step t.  xs is
 * the dense [T,B,H] array with anything finite (zeros) in the dead places;
 * hsss/csss are written for the live (t, row) pairs, what the other places
 * hold afterwards is unspecified.  32-row blocks that have ended are skipped
 * by the persistent kernel; the streamed stacks of the other hidden sizes
 * compute the live rows of every step only; the fp32-MFMA fallback computes
 * everything.
 * dilations: host array or NULL (all 1).  Replaces the shrinking batch of
 * batched_cell (examples/stacked_rnn/stacked_rnn.py:45-51, hs_prev[0:xs.length])
 * over the layout of gen_dataset_time_major (examples/utils/data_utils.py:42-66).
 */
int ftk_stacked_lstm_ragged_f32(const float* xs, const float* WU,
                                const float* bias, const int* dilations,
                                const int* active_rows, float* hsss,
                                float* csss, int L, int T, int B, int H,
                                void* workspace, size_t workspace_bytes,
                                ftk_stream_t stream);

/*
 * The stack with fp16 storage, the numeric form of the reference's CuTe LSTM:
 * xs [T,B,H], WU [L,2H,4H], hsss, csss [L,T,B,H] all fp16 (h and c are rounded
 * to fp16 when written, and read back rounded), bias [L,4H] fp32 or NULL, gate
 * sums accumulated in fp32.  H%32==0.  H = 512 and H = 256 with even B, the
 * first two hidden sizes of the reference's sweep, run in the persistent
 * kernel: fp16 weights of H = 512 take the registers the fp32 weights of
 * H = 256 take; stacks deeper than the chip holds at once (16 layers of
 * H = 512, 32 of H = 256 on 256 compute units) run as consecutive launches.
 * Every other shape (H = 1024, the third size of the sweep, among them) does
 * not fit on chip: its weights are streamed, one launch of the fp16 cell
 * kernel per stage of independent cells, on the rows that live at the cell's
 * step (which is also the faster way for H = 512 stacks of more than 16
 * layers, unless active_rows is given; FTK_LSTM_F16_STREAM=1 / 0 forces
 * either); the
 * workspace then takes a re-laid copy of WU (ftk_stacked_lstm_f16_workspace_bytes
 * says how much for a shape).
 * dilations, active_rows: host arrays or NULL, as above.
 * Replaces StackedLstmRegion1/2/3 with Element = half as instantiated by
 * benchmarks/rnn/fractaltensor/cute_stacked_lstm/stacked_lstm.cu:16-19,59-155
 * (run_bench<32, 64, 256, 256>, <32, 64, 256, 512>, <32, 64, 256, 1024>, :185-187).
 */
size_t ftk_stacked_lstm_f16_workspace_bytes(int L, int T, int B, int H);
int ftk_stacked_lstm_f16(const void* xs, const void* WU, const float* bias,
                         const int* dilations, const int* active_rows,
                         void* hsss, void* csss, int L, int T, int B, int H,
                         void* workspace, size_t workspace_bytes,
                         ftk_stream_t stream);

/*
 * How the persistent kernel of the fp32 entry points above forms the products
 * of the gate GEMM.  FTK_LSTM_PRODUCTS_F32: one v_mfma_f32_32x32x2_f32 per
 * product.  FTK_LSTM_PRODUCTS_F16X3 (the default): every fp32 operand is cut
 * into an fp16 value and an fp16 remainder under a power-of-two scale shared
 * by its weight column / activation row, three fp16 MFMAs with fp32
 * accumulation take the place of the fp32 one and only the remainder x
 * remainder term (2^-22 of a product) is dropped; inputs, state, outputs and
 * accumulation stay fp32.  The streamed path of the other hidden sizes forms
 * the same three products (as three k chunks per chunk of the contraction)
 * and keeps the remainders unscaled.  The environment variable FTK_LSTM_PRODUCTS=f32 or
 * =f16x3 sets the initial mode.  A tuning control of this library: the
 * reference has one fp32 (cuBLAS) and one fp16 (CuTe) LSTM and no switch.
 */
#define FTK_LSTM_PRODUCTS_DEFAULT (-1)
#define FTK_LSTM_PRODUCTS_F32 0
#define FTK_LSTM_PRODUCTS_F16X3 1
/* The process-wide default (initially F16X3 or what FTK_LSTM_PRODUCTS says).  One
 * plain int shared by every thread: set it before other threads call the LSTM
 * entry points, or choose per call through ftk_stacked_lstm_opts_f32 instead. */
int ftk_lstm_set_products(int mode);
int ftk_lstm_get_products(void);

/*
 * The fp32 stack with everything per call: dilations and active_rows as in
 * the entry points above (host arrays, either may be NULL) plus
 *   products:   FTK_LSTM_PRODUCTS_F32 / _F16X3, or _DEFAULT for the process-wide
 *               mode.  With F16X3 non-finite inputs give NaN where fp32
 *               arithmetic would give +-inf (the remainder plane of an infinite
 *               value is inf - inf);
 *   spin_limit: polls a bounded wait of the persistent kernel makes before it
 *               gives up, 0 = the default (2^22, seconds).
 * options == NULL means {DEFAULT, 0}.  No counterpart in the reference.
 */
typedef struct ftk_lstm_options {
  int products;
  int spin_limit;
} ftk_lstm_options;
int ftk_stacked_lstm_opts_f32(const float* xs, const float* WU, const float* bias,
                              const int* dilations, const int* active_rows,
                              float* hsss, float* csss, int L, int T, int B,
                              int H, const ftk_lstm_options* options,
                              void* workspace, size_t workspace_bytes,
                              ftk_stream_t stream);

/*
 * Whether the last stacked-LSTM call that was given `workspace` ran to the end.
 * The persistent kernel synchronises its workgroups through counters in the
 * workspace; every wait is bounded, and a wait that runs out (workgroups not
 * co-resident, a lost device) sets the status word -- the first int of every
 * LSTM workspace, zeroed by every call -- and drains the launch, leaving
 * hsss / csss partly unwritten.  The entry points have returned 0 by then:
 * they are asynchronous.  This call WAITS for `stream`, reads the word and
 * returns FTK_OK or FTK_ERR_TIMEOUT.  Callers must check it (here, or by
 * reading the word themselves after synchronising) before trusting the
 * outputs of ftk_stacked_lstm_f32 / _dilated_ / _ragged_ / _opts_ / _f16.
 * workspace == NULL: the built-in scratch of ftk_stacked_lstm_noalloc_f32 on
 * the current device (FTK_ERR_INVALID_ARGUMENT if that has never run there).
 * No counterpart in the reference, whose launches do not wait for each other.
 */
int ftk_stacked_lstm_status(const void* workspace, ftk_stream_t stream);

/*
 * Waits for `stream`; 1 if the last fp32 stacked-LSTM call given this
 * workspace ran on split products (FTK_LSTM_PRODUCTS_F16X3) and met hidden
 * states too small for them, 0 if not, negative on error.  Split products
 * hand h from cell to cell as two fp16 planes under a fixed scale (|h| < 1):
 * the results are accurate to a few 1e-7 of the LARGEST |h|, but a non-zero
 * |h| below 2^-26 reaches the cells that read it with fewer than 13 bits of
 * its own, and below about 2^-38 as zero.  One such value beside larger ones
 * is harmless (its error is 2^-38 in absolute terms); reported is a row in
 * which four neighbouring units are all that small and not all zero.
 * A stack whose upper layers fade towards zero (small weights, no bias)
 * is then exact relative to the whole output and
 * inexact relative to those layers; a caller that needs every layer accurate
 * to its own size repeats the call with FTK_LSTM_PRODUCTS_F32 when this
 * returns 1.  No counterpart in the reference (its CuTe stack is fp16
 * throughout, benchmarks/rnn/fractaltensor/cute_stacked_lstm/stacked_lstm.cu:16-19).
 */
int ftk_stacked_lstm_small_states(const void* workspace, ftk_stream_t stream);

/*
 * ftk_stacked_lstm_opts_f32 with fp32 products for callers that cannot
 * allocate device memory or pass a workspace: tight serving loops, harnesses
 * that forbid hipMalloc, code that prepares a HIP graph.  No counterpart in
 * the reference.  The first call on a device does set-up that is no
 * allocation but is no stream work either (the scratch's address, a function
 * attribute, an occupancy query): make one call per device before any region
 * that must hold nothing but launches.  The launch is a cooperative one
 * (hipLaunchCooperativeKernel); that a stream capture records it has not been
 * exercised here.  Same operands and results as ftk_stacked_lstm_opts_f32
 * with {FTK_LSTM_PRODUCTS_F32, 0} and no active_rows; H must be 256, and the
 * status block, flags and trace of the launch (about 64*L*T*ceil(B/32) +
 * 64*T*ceil(B/32) + 256 bytes) must fit the library's built-in scratch of
 * 2 MiB per device (config 4, L32 T64 B256: 1.03 MiB), else
 * FTK_ERR_UNSUPPORTED_SHAPE; likewise when L layers do not fit the device in
 * one persistent launch.  The call allocates nothing, frees nothing and waits
 * for nothing.  Every call on a device shares that device's scratch: calls
 * that overlap on one device (two streams, two threads) race; calls on one
 * stream are safe.  ftk_stacked_lstm_status(NULL, stream) reads the status
 * word of the current device's scratch.
 */
int ftk_stacked_lstm_noalloc_f32(const float* xs, const float* WU,
                                 const float* bias, const int* dilations,
                                 float* hsss, float* csss, int L, int T, int B,
                                 int H, ftk_stream_t stream);

/*
 * The same stack evaluated as one batched fused-cell launch per wavefront
 * diagonal (no persistent kernel, no workspace); any H%32==0.  This is the
 * launch structure of StackedLstmRegion3 (region3.h:50-103) and the fallback
 * of the two entry points above.  dilations: host array or NULL (all 1).
 */
int ftk_stacked_lstm_wavefront_f32(const float* xs, const float* WU,
                                   const float* bias, const int* dilations,
                                   float* hsss, float* csss, int L, int T,
                                   int B, int H, ftk_stream_t stream);

/*
 * Stacked grid RNN, fp32: D blocks over an L1 x L2 grid of positions, two tanh
 * cells per position that share the state of both directions,
 *   s = [h_x(d,i-1,j) | h_y(d,i,j-1)]  (zeros outside the grid),
 *   h_x(d,i,j) = tanh(x_in @ Wx[d] + s @ Ux[d] + bx[d]),
 *   h_y(d,i,j) = tanh(y_in @ Wy[d] + s @ Uy[d] + by[d]),
 * where (x_in, y_in) = (h_x, h_y)(d-1,i,j) for d > 0 and, in the first block,
 * (xs[i], ys[j]) (crossed = 0: xs [L1,B,H], ys [L2,B,H]) or (xs[j], ys[i])
 * (crossed = 1: xs [L2,B,H], ys [L1,B,H]).  W* [D,H,H], U* [D,2H,H], biases
 * [D,bias_rows,H] with bias_rows 1 or B, or both NULL; hsss
 * [D,L1,L2,2,B,H] receives h_x (index 0) and h_y (index 1) of every position
 * and is also where the kernel reads the neighbours back, so no gather or
 * scatter buffers exist.  One launch per plane d+i+j.  H%32==0.  Passing the
 * same pointers for both directions gives the shared-parameter model.
 * workspace: 16-byte aligned device memory of ftk_grid_rnn_workspace_bytes(D, H)
 * bytes (half of it suffices with shared parameters) into which every call
 * first re-lays the parameters in the order the kernel's lanes read them; with
 * NULL or less room the kernel reads the parameters where they lie (about 10 %
 * slower).
 * Replaces the eight wavefront regions of
 * benchmarks/rnn/fractaltensor/grid_lstm/regions/region1.h-region8.h (general
 * case region8.h:61-310: gather, VanillaRNNCellBMM utils.h:671-700, scatter;
 * crossed = 0, shared parameters, bias_rows = B, stacked_grid_rnn.cu:31-41) and
 * is the device form of examples/grid_rnn/grid_rnn.py:40-137 (crossed = 1,
 * parameters per direction, bias_rows = 1).  Unlike utils.h:650, a plane that
 * holds a single position still gets its bias and tanh.
 */
size_t ftk_grid_rnn_workspace_bytes(int D, int H);
int ftk_grid_rnn_f32(const float* xs, const float* ys, const float* Wx,
                     const float* Ux, const float* bx, const float* Wy,
                     const float* Uy, const float* by, float* hsss, int D,
                     int L1, int L2, int B, int H, int bias_rows, int crossed,
                     void* workspace, size_t workspace_bytes,
                     ftk_stream_t stream);

/*
 * Embedding lookup, the step that feeds the LSTM in the reference's RNN
 * programs: out[i, :] = table[ids[i], :] for i < n.  table [V,E] fp32, ids [n]
 * int32 (ids_are_64bit = 0) or int64 (1) on the device, out [n,E]; E%4==0.
 * An id outside [0,V) zero-fills its row and adds 1 to *bad_ids (a device int
 * the caller has zeroed, or NULL) instead of reading out of bounds; the Python
 * side turns a non-zero count into the IndexError the reference raises.
 * Replaces ops.map(lambda word: ops.index(ops.slices(embedding, dim=0), word), ws)
 * (examples/stacked_rnn/rnn_utils.py:81-90; Index, access.py:36-58).
 */
int ftk_embedding_gather_f32(const float* table, const void* ids,
                             int ids_are_64bit, float* out, long long n, int V,
                             int E, int* bad_ids, ftk_stream_t stream);

/* ------------------------------------------------------------ B2B GEMM -- */

/*
 * G independent problems D = (A @ B) @ C, fp16 storage, fp32 accumulation,
 * intermediate A@B rounded to fp16 in registers between the two products.
 * A [G,M,K] row-major; B stored [G,N,K] (= K x N column-major); C stored
 * [G,P,N] (= N x P column-major); D [G,M,P] row-major -- the layouts of
 * kaleido/core/operators/tests/b2b_gemm_test_utils.h:3-9.
 * Needs K%16==0, N%32==0, P%32==0, any M.  K of 32, 64, 96 or 128 with B and a
 * 128-column tile of C small enough for LDS (N up to 256 at K=128, 512 at
 * K=64) runs on the fused kernels that keep B and C on chip; every other
 * shape (N <= 2048), the reference test's [192,704]x[704,448]x[448,832]
 * (kaleido/core/operators/tests/test_b2b_gemm.cu:137-149) included, on a
 * general kernel that streams B and C.
 * Replaces B2BGemm::operator() (kaleido/core/device/kernels/gemm.h:235-269,
 * KeBack2BackGemm cutlass_wmma.h:441-540); the reference has no batch
 * dimension, G maps to independent workgroups.
 */
int ftk_b2b_gemm_f16(const void* A, const void* B, const void* C, void* D,
                     int G, int M, int N, int K, int P, ftk_stream_t stream);

/*
 * 1 when ftk_b2b_gemm_f16 takes products of this shape on the current device
 * (any G and M), 0 when it would return FTK_ERR_UNSUPPORTED_SHAPE or no device
 * can be queried.  For callers that choose between the fused product and two
 * plain ones before they call, as kaleido's `(a @ b) @ c` does
 * (Tensor.__matmul__, kaleido/frontend/tensor.py:218-220); the reference's
 * B2BGemm fixes its shapes at compile time (gemm_kernel_traits.h:214-283).
 */
int ftk_b2b_gemm_f16_supported(int N, int K, int P);

/*
 * The same product with every operand row-major, the layout an operator
 * program's (a @ b) @ c has: A [G,M,K], B [G,K,N], C [G,N,P], D [G,M,P].
 * B and C are staged as they are and transposed on the way from LDS to the
 * matrix unit.  Built for the shapes of the eight-wave kernel: K and N in
 * {64, 128}, P%128==0 (anything else: FTK_ERR_UNSUPPORTED_SHAPE; transpose B
 * and C once and call ftk_b2b_gemm_f16).  No counterpart in the reference,
 * whose B2BGemm takes column-major B and C only (gemm_kernel_traits.h:261-267);
 * it is what kaleido's `(a @ b) @ c` (Tensor.__matmul__, kaleido/frontend/tensor.py:218-220) maps to.
 */
int ftk_b2b_gemm_rowmajor_f16(const void* A, const void* B, const void* C,
                              void* D, int G, int M, int N, int K, int P,
                              ftk_stream_t stream);

/* ------------------------------------------------------------ plain GEMM -- */

/*
 * C = A @ B, fp16 storage, fp32 accumulation, every operand row-major:
 * A [M,K], B [K,N], C [M,N]; the batched form takes G independent problems
 * A [G,M,K], B [G,K,N], C [G,M,N].  Needs N%128==0, K%32==0 and 16-byte
 * aligned A, B, C.  N%256==0 runs
 * on a kernel built for the product (256 x 256 outputs per workgroup, one wave
 * per SIMD with 128 x 128 of them, k chunks of 32 through all 160 KB of LDS,
 * A a whole cache line per row at a time, B transposed between LDS and the
 * matrix unit; any M); other widths on the
 * streaming LSTM cell kernel without the cell.  Stands in for
 * KeCuteGemm / KeBatchedCuteGemm / KeGemmPipelined
 * (kaleido/core/device/kernels/cutlass_wmma.h:116,186,259; functors CuteGemm,
 * GemmPipelined gemm.h:152,201 and batched_gemm.h:84) behind ops.mm (MatMul,
 * kaleido/frontend/operations/tensor/arithmetic/contraction.py:21).
 */
int ftk_gemm_f16(const void* A, const void* B, void* C, int M, int N, int K,
                 ftk_stream_t stream);
int ftk_batched_gemm_f16(const void* A, const void* B, void* C, int G, int M,
                         int N, int K, ftk_stream_t stream);

/* ------------------------------------------------------ flash attention -- */

/*
 * O = softmax(Q K^T * scale) V per (batch, head), non-causal, fp16 storage,
 * fp32 accumulation, online softmax (running max / sum) in registers.
 * Q,O [B,Hd,Sq,D]; K,V [B,Hd,Skv,D].  D == 128, 96, 64 or 32; any Sq, Skv >= 1 (the
 * last, partial blocks of queries and keys are masked).
 * Replaces the map/reduce program flash_attention
 * (examples/flash_attention/flash_attention.py:14-91); the reference has no
 * device kernel for it.
 */
int ftk_flash_attn_f16(const void* Q, const void* K, const void* V, void* O,
                       int B, int Hd, int Sq, int Skv, int D, float scale,
                       ftk_stream_t stream);

/*
 * The same call with a workspace, for grids that do not fill the chip: when
 * batch x heads x (query blocks of 128 rows) covers less than half of the
 * compute units and there are at least 2048 keys, the keys are cut into up to
 * 64 contiguous parts, every part runs as a workgroup of its own and leaves
 * (reference maximum, sum of exponentials, unnormalised O) in the workspace,
 * and a second launch merges the parts by the rule of an online softmax
 * (kaleido/core/device/kernels/online_softmax.h:27-30).
 * ftk_flash_attn_f16_workspace_bytes is 0 for shapes that are not split;
 * without a sufficient workspace the call is ftk_flash_attn_f16.  The
 * reference has no device kernel for this program.
 */
size_t ftk_flash_attn_f16_workspace_bytes(int B, int Hd, int Sq, int Skv, int D);
int ftk_flash_attn_ws_f16(const void* Q, const void* K, const void* V, void* O,
                          int B, int Hd, int Sq, int Skv, int D, float scale,
                          void* workspace, size_t workspace_bytes,
                          ftk_stream_t stream);

/*
 * The same attention with fp32 Q, K, V and O, [B,Hd,S,D] row-major, D of 32,
 * 64, 96 or 128: the element type of the reference's program
 * (examples/flash_attention/flash_attention.py:14-91 on kaleido.float32
 * blocks, flash_attention_utils.py:20-24; batch 2 x 8 heads x 1024 x 32 at
 * :96-110).  Products run on the fp16 matrix pipe as three fp16 products of
 * split operands with fp32 accumulation (a row of Q, all of K and all of V of
 * a (batch, head) each share a power-of-two scale), the softmax state is fp32:
 * results agree with a float64 evaluation to a few 1e-6 of the largest |O|.
 * Q, K, V, O 16-byte aligned.  Non-finite inputs give NaN.  The workspace (ftk_flash_attn_f32_workspace_bytes,
 * about the size of K and V together, 256-byte aligned) holds their split
 * planes (Q is split in the attention kernel's registers); three small
 * launches precede the attention kernel.  The reference has no device kernel
 * for this program.
 */
size_t ftk_flash_attn_f32_workspace_bytes(int B, int Hd, int Sq, int Skv, int D);
int ftk_flash_attn_f32(const float* Q, const float* K, const float* V, float* O,
                       int B, int Hd, int Sq, int Skv, int D, float scale,
                       void* workspace, size_t workspace_bytes,
                       ftk_stream_t stream);

/*
 * Windowed attention, fp32: token t of each of the G sequences attends to the
 * `window` (odd) positions t - half + k*dilation, k = 0..window-1,
 * half = (window-1)*dilation/2, and to the R further positions
 * extra_idx[g, t, 0..R-1] (int32 on the device; NULL with R = 0):
 *   O[g,t] = softmax(scale * Q[g,t] . K[g,P]^T) . V[g,P],  P = window ++ extra.
 * Q, K, V, O [G,S,D] row-major, 16-byte aligned; D%4==0, D <= 1024.  Window
 * positions past an end wrap as the reference's shifted_slide wraps them:
 * p >= S -> p - S, p < 0 -> p + S - 1 (kaleido/frontend/operations/access.py:
 * 384-390; one short of circular at the left end, kept as it is).  An
 * extra_idx entry outside [0,S) is clamped rather than read out of bounds;
 * the Python side raises IndexError before the call, as indexing a
 * FractalTensor does.
 * Replaces, per head, ops.shifted_slide(ops.zip(key, value), window_size,
 * dilation) followed by the map of sparse_attn over the tokens
 * (examples/sparse_attention/sparse_attention.py:25-38, 51-53, 69-71:
 * softmax(q @ [windowed ++ random keys]^T) @ [windowed ++ random values],
 * scale = 1); the reference has no device kernel for it.
 */
int ftk_windowed_attn_f32(const float* Q, const float* K, const float* V,
                          const int* extra_idx, float* O, int G, int S, int D,
                          int window, int dilation, int R, float scale,
                          ftk_stream_t stream);

/*
 * Row softmax through an online (max, denominator) scan, fp32, [rows, cols].
 * Replaces OnlineNormalizedSoftmaxOp
 * (kaleido/core/operators/online_softmax_op.cu:14-36,
 * KeOnlineNormalizedSoftMax kaleido/core/device/kernels/online_softmax.h:176-183).
 */
int ftk_online_softmax_f32(const float* x, float* y, int rows, int cols,
                           ftk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FTK_H_ */
