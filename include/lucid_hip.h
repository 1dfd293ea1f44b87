/*
 * lucid_hip.h - C ABI of the MI355X (gfx950) backend for Lucid's int8
 * quantized-inference path.
 *
 * The library is the drop-in for the part of Lucid's backend seam
 * (lucid/_C/backend/IBackend.h:226-2239, selected through
 * lucid/_C/backend/Dispatcher.h:90-94) that lucid.quantization and
 * lucid.nn.quantized reach.  Lucid composes quantize / dequantize /
 * fake_quantize out of five to seven elementwise virtuals and runs quantized
 * Linear / Conv2d as dequantize + float GEMM + fake_quantize; this ABI exposes
 * each of those composites as ONE fused entry point instead, which is what a
 * HIP backend registered beside CpuBackend (CpuBackend.h:13835-13842) and
 * GpuBackend (GpuBackend.h:7782-7787) would bind.
 *
 * Conventions
 *   - every function returns an lq_status (0 = ok); lq_last_error() returns the
 *     thread-local message of the last failure.  Status values mirror Lucid's
 *     exception family (lucid/_C/core/Error.h:63-495).
 *   - all tensor pointers are DEVICE pointers to contiguous row-major data
 *     unless a parameter is documented as host memory.
 *   - lq_dtype values equal Lucid's Dtype enum order (lucid/_C/core/Dtype.h).
 *   - a tensor is described around its channel axis as [outer][C][inner]
 *     (the broadcast of lucid/quantization/_functional.py:45-54); per-tensor
 *     parameters use C = 1.
 *   - launches are asynchronous on `stream` (a hipStream_t; NULL = the default
 *     stream).  lq_sync / lq_d2h synchronise.
 *   - reductions, gathered matrices and the split-K GEMM use scratch owned by
 *     the library, one buffer per (device, stream): calls on different streams
 *     do not share scratch and may overlap; calls on one stream are ordered by
 *     it.  The functions are re-entrant (Lucid's dispatcher is read-only and
 *     concurrent-safe after start-up, lucid/_C/backend/Dispatcher.h:49-52).
 *   - an output that is also read by the same call (out == residual, or
 *     out == join.q of lq_qlinear_i8 / lq_qconv2d_i8) is allowed: every element
 *     is read before it is written by the same lane.  The first-call tile
 *     tuner is skipped for such calls (it would apply the operand repeatedly).
 */
#ifndef LUCID_HIP_H
#define LUCID_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LQ_VERSION 3

typedef enum {
    LQ_OK = 0,
    LQ_ERR_VALUE = 1,            /* ValueError: bad argument value            */
    LQ_ERR_SHAPE = 2,            /* ShapeMismatch      (Error.h)              */
    LQ_ERR_DTYPE = 3,            /* DtypeMismatch                             */
    LQ_ERR_DEVICE = 4,           /* DeviceMismatch                            */
    LQ_ERR_OOM = 5,              /* OutOfMemory                               */
    LQ_ERR_GPU_NOT_AVAILABLE = 6,/* GpuNotAvailable                           */
    LQ_ERR_NOT_IMPLEMENTED = 7,  /* NotImplementedError                       */
    LQ_ERR_INTERNAL = 8          /* LucidError (any other HIP failure)        */
} lq_status;

/* lucid/_C/core/Dtype.h enum order */
typedef enum {
    LQ_BOOL = 0, LQ_I8 = 1, LQ_I16 = 2, LQ_I32 = 3, LQ_I64 = 4,
    LQ_F16 = 5, LQ_F32 = 6, LQ_F64 = 7, LQ_C64 = 8, LQ_BF16 = 9, LQ_C128 = 10
} lq_dtype;

typedef void* lq_stream; /* hipStream_t */
typedef void* lq_event;  /* hipEvent_t  */

/* ------------------------------------------------------------------ runtime */
/* Storage / transfer: IBackend::from_cpu (IBackend.h:259), to_cpu (:1370),
 * and the allocator (lucid/_C/core/Allocator.h). */
int lq_version(void);
const char* lq_last_error(void);
int lq_device_count(int* count);
int lq_init(int device);
int lq_device_name(char* buf, size_t buflen);
/* Device memory comes from a caching pool (freed blocks are reused without
 * going back to the driver); lq_empty_cache returns cached blocks to it. */
int lq_alloc(void** ptr, size_t nbytes);
int lq_free(void* ptr);
int lq_empty_cache(void);
int lq_memory_stats(size_t* bytes_in_use, size_t* bytes_reserved); /* MemoryStats, bind_tensor.cpp */
/* Free and total bytes of the current device as the driver reports them (hipMemGetInfo): unlike
 * lq_memory_stats this sees every allocation, the library's own scratch included. */
int lq_device_memory_info(size_t* free_bytes, size_t* total_bytes);
int lq_h2d(void* dst_dev, const void* src_host, size_t nbytes, lq_stream stream);
int lq_d2h(void* dst_host, const void* src_dev, size_t nbytes, lq_stream stream);
int lq_d2d(void* dst_dev, const void* src_dev, size_t nbytes, lq_stream stream);
/* `rows` rows of row_bytes each between two pitched device buffers (a column slice of a
 * matrix: one direction's half of a bidirectional LSTM output, a channel slice). */
int lq_d2d_rows(void* dst_dev, size_t dst_pitch, const void* src_dev, size_t src_pitch, size_t row_bytes,
                size_t rows, lq_stream stream);
int lq_fill_bytes(void* dst_dev, int value, size_t nbytes, lq_stream stream);
int lq_sync(lq_stream stream);
int lq_stream_create(lq_stream* stream);
/* A stream that does not synchronise implicitly with the default stream (hipStreamNonBlocking,
 * default priority): work on several of them overlaps even while the default stream is in use;
 * order them with events (lq_event_record / lq_stream_wait_event). */
int lq_stream_create_nonblocking(lq_stream* stream);
int lq_stream_destroy(lq_stream stream);
int lq_event_create(lq_event* ev);
int lq_event_destroy(lq_event ev);
int lq_event_record(lq_event ev, lq_stream stream);
/* Work queued on `stream` after this call waits for `ev` (hipStreamWaitEvent): the
 * fork / join of forwards that run on several streams at once. */
int lq_stream_wait_event(lq_stream stream, lq_event ev);
int lq_event_sync(lq_event ev);
int lq_event_elapsed_ms(lq_event start, lq_event stop, float* ms);

/* HIP graphs: capture everything launched on `stream` between begin and end
 * (a created stream, not the default one), then replay it with one launch -
 * for launch-bound inference loops (a quantized ResNet-50 forward is ~75 short
 * kernels).  Memory allocated during capture stays reserved for the graph until
 * lq_graph_destroy.  No counterpart in Lucid (its Metal backend batches lazily
 * through MLX instead). */
int lq_graph_begin(lq_stream stream, int* graph_id);
int lq_graph_end(lq_stream stream, int graph_id);
int lq_graph_launch(int graph_id, lq_stream stream);
int lq_graph_destroy(int graph_id);

/* Op registry: OpSchema{name, version, deterministic}
 * (lucid/_C/core/OpSchema.h, OpRegistry.h:55,158-164). */
int lq_op_count(void);
int lq_op_info(int index, const char** name, int* version, int* deterministic);

/* Synthetic-data helper for benchmarks: fills x[n] with N(0,1) samples from a
 * counter-based generator; a fraction `outlier_prob` of them is multiplied by
 * `outlier_gain`.  No counterpart in Lucid (its RNG is off this path). */
int lq_fill_normal(float* x, size_t n, uint64_t seed, float outlier_prob, float outlier_gain,
                   lq_stream stream);
int lq_fill_uniform_i8(int8_t* x, size_t n, uint64_t seed, int lo, int hi, lq_stream stream);
/* ---- quantized module breadth (lucid/nn/quantized/{sparse,activation,conv_transpose}.py,
 * dynamic/rnn.py) ---- */

/* out2[0] = min, out2[1] = max of an int32 / int64 index tensor (n > 0): the range
 * check of lucid/nn/functional/sparse.py:17-71 without a host copy of the indices. */
int lq_index_minmax(const void* idx, int idx_is_64, size_t n, long long* out2, lq_stream stream);

/* nnq.Embedding.forward (sparse.py:128-134 = dequantize + F.embedding,
 * CpuBackend.h:8970-9010): out[i, :] = (table[idx[i], :] - zp[idx[i]]) * scale[idx[i]],
 * zeros where idx[i] == padding_idx >= 0 (pass -1 for none).  table int8
 * [num_embeddings, dim], per-row scale / zp; only the rows asked for are read.  Ids
 * outside the table give zeros (callers check the range first, as Lucid does). */
int lq_embedding_i8(const int8_t* table, const float* scale, const float* zp, int num_embeddings, int dim,
                    const void* idx, int idx_is_64, size_t n_idx, int padding_idx, float* out,
                    lq_stream stream);

/* nnq.EmbeddingBag.forward (sparse.py:270-279 = dequantize + F.embedding_bag,
 * CpuBackend.h:5989-6088): bag b pools the decoded rows of idx[offsets[b] .. offsets[b+1])
 * (the last bag runs to n_idx); offsets == NULL: idx is bags x fixed_len, one bag per row.
 * mode 0 sum (rows added in index order), 1 mean (divided by the rows added, if any),
 * 2 max (an empty bag gives zeros); padding_idx (-1 for none) and ids outside the table
 * are skipped.  out float32 [bags, dim]. */
int lq_embedding_bag_i8(const int8_t* table, const float* scale, const float* zp, int num_embeddings, int dim,
                        const void* idx, int idx_is_64, size_t n_idx, const void* offsets, int offsets_is_64,
                        int fixed_len, int bags, int mode, int padding_idx, float* out, lq_stream stream);

/* Activations of lucid/nn/quantized/activation.py: kind 0 sigmoid, 1 hardswish,
 * 2 hardsigmoid, 3 tanh, 4 elu(alpha), 5 leaky_relu(alpha = negative slope); float32
 * formulas of CpuBackend.h:1049-1060,1722-1723,1783-1785,2001-2002,2064-2065.
 * lq_act_f32: out = act(x), then fake-quantized to (out_scale, out_zp, [qmin, qmax])
 * when fake_quantize_out != 0 (_QuantizedActivation.forward, activation.py:44-53).
 * lq_act_requant_i8: the same for an input carried as codes on a per-tensor grid,
 * output as codes: out = requantize(act(dequantize(q))) element by element. */
int lq_act_f32(int kind, float alpha, const float* x, float* out, size_t n, int fake_quantize_out,
               const float* out_scale, const float* out_zp, int out_qmin, int out_qmax, lq_stream stream);
int lq_act_requant_i8(int kind, float alpha, const int8_t* q, int q_offset, const float* scale, const float* zp,
                      size_t n, const float* out_scale, const float* out_zp, int out_qmin, int out_qmax,
                      int out_offset, int8_t* out, lq_stream stream);

/* Zero insertion for nnq.ConvTranspose2d (conv_transpose.py): NHWC codes [B, H, W, C] ->
 * [B, (H-1)*stride_h + 1 + extra_h, (W-1)*stride_w + 1 + extra_w, C]; input pixels land on
 * multiples of the stride, every other byte is `fill` (the stored code of real zero).
 * A stride-1 lq_qconv2d_i8 of the result with the flipped, transposed kernel and padding
 * dilation*(k-1) - p is the transposed convolution (extra = output_padding). */
int lq_dilate_nhwc_i8(const int8_t* x, int B, int H, int W, int C, int stride_h, int stride_w, int extra_h,
                      int extra_w, int fill, int8_t* out, lq_stream stream);

/* One LSTM time step after the two gate products (CpuBackend.h:13456-13506; gate order
 * i, f, g, o): raw = gates_x + gates_h + bias (bias = b_ih + b_hh or NULL, [4*hidden]),
 * c_out = sigmoid(f)*c_in + sigmoid(i)*tanh(g), h_out = sigmoid(o)*tanh(c_out); h is also
 * written to y (row stride y_ld) when y != NULL.  gates_x: this step's rows of x W_ih^T,
 * row stride gates_x_ld floats (the product is taken once over all time steps);
 * gates_h float32 [batch, 4*hidden] contiguous. */
int lq_lstm_cell_f32(const float* gates_x, size_t gates_x_ld, const float* gates_h, const float* bias,
                     const float* c_in, int batch, int hidden, float* h_out, float* c_out, float* y,
                     size_t y_ld, lq_stream stream);

/* Self-test of the tile kernels' requantize arithmetic.  Their epilogue computes
 * clamp(rint(x / scale) + zp, qmin, qmax) mostly without dividing (x * (1/scale),
 * accepted when it lies clear of every rounding boundary, the IEEE quotient
 * otherwise), with a ReLU directly before it (relu != 0) folded into the lower
 * clamp bound, ahead of a fused join as the code minus zp from shifted bounds,
 * and for packing as the code shifted into 0..255.  This runs those forms of
 * the routine and the plain [max(x, 0),]
 * divide-round-add-clamp of quantize (lucid/quantization/_functional.py:164-182)
 * on every float32 bit pattern in [first_bits, first_bits + count) and counts the
 * patterns whose stored code would differ (*mismatches, must be 0) and those
 * that took the dividing branch (*divided).  Both counters are device memory
 * (8 bytes each).  No counterpart in Lucid. */
int lq_selftest_requant_route(float scale, float zp, int qmin, int qmax, int relu,
                              unsigned long long first_bits, unsigned long long count,
                              unsigned long long* mismatches, unsigned long long* divided,
                              lq_stream stream);

/* Matrix-core rate probe for roofline accounting: 2 blocks per CU, each
 * wavefront issuing `iters` rounds of eight v_mfma_i32_32x32x32_i8 on eight
 * independent accumulators, operands taken from a[] / b[] (at least 32 KiB
 * each, 16-byte aligned) and rotated so that operand bits toggle as they do in
 * a GEMM over that data; no LDS or memory traffic in the loop.  *ops receives
 * the integer operations launched (2*32*32*32 per instruction); time the call
 * with events to get the rate the matrix cores sustain under the power limit
 * for these operand statistics.  sink: one int of device memory.  No
 * counterpart in Lucid. */
int lq_probe_mfma_i8(const int8_t* a, const int8_t* b, size_t nbytes, int iters, int* sink,
                     double* ops, lq_stream stream);
/* The same probe with the instruction and the register walk of the large-GEMM kernel: each
 * wavefront keeps 4 x 11 tiles of v_mfma_i32_16x16x64_i8 (2*16*16*64 operations each) and visits
 * them column by column, alternating the row order; at least 44 KiB per operand.  The two
 * instructions sustain different rates on the same operand data under the power limit. */
int lq_probe_mfma_i8_k64(const int8_t* a, const int8_t* b, size_t nbytes, int iters, int* sink,
                         double* ops, lq_stream stream);
/* Plain device copy kernel (n bytes, 16-byte vectors): the calibration
 * workload for hardware-counter scaling. */
int lq_copy_kernel(void* dst, const void* src, size_t nbytes, lq_stream stream);

/* ---------------------------------------------------------- engine primitives */
/* The IBackend calls that Lucid's quantization composites are written in, one kernel
 * each, on contiguous device buffers of n elements - what an unmodified
 * clip(round(x / s) + z, qmin, qmax).to(int8) (lucid/quantization/_functional.py:180),
 * (q.to(float32) - z) * s (_functional.py:281) or an observer's min / max dispatches to
 * when its tensors live on this device.  The fused lq_quantize / lq_dequantize /
 * lq_fake_quantize / lq_minmax give the same bits in one pass and are what the modules
 * use; these are the slow, call-for-call route and the specification of the fused ones.
 *   lq_add/sub/mul/div_f32     IBackend::add/sub/mul/div (IBackend.h:370-373; IEEE float32,
 *                              division as vDSP_vdiv, Vdsp.cpp:47-48); lq_add_f32 is declared
 *                              with the float32 network kernels below
 *   lq_maximum/minimum_f32     IBackend::maximum/minimum (IBackend.h:433-434): a NaN in either
 *                              operand gives NaN (vDSP_vmax / vDSP_vmin, Vdsp.cpp:140-151)
 *   lq_round_f32               IBackend::round (IBackend.h:474): ties to even (vvnintf,
 *                              Vforce.cpp:136)
 *   lq_clip_f32                IBackend::clip (IBackend.h:1232): bounds cast to float, NaN
 *                              passes through (CpuBackend.h:6880-6891)
 *   lq_astype                  IBackend::astype / cast (IBackend.h:2121,1235): static_cast
 *                              between LQ_I8 / I16 / I32 / F16 / F32 (CpuBackend.h:6214-6236);
 *                              float -> integer saturates at int32 and maps NaN to 0 (both
 *                              undefined in C), then truncates to the width
 *   lq_broadcast_f32           the materialised broadcast of a per-channel operand,
 *                              out[o,c,i] = src[c] (kernel/BinaryKernel.h:591-606)
 *   lq_reduce_minmax           IBackend::reduce_min + reduce_max over `axes` (IBackend.h:689-692;
 *                              n_axes == 0 reduces everything), NaN-propagating
 *                              (Reduce.cpp:87-125); mn / mx hold one float per kept
 *                              element in row-major order.  The reduced axes must merge into
 *                              one run of neighbouring dimensions or into the two ends of
 *                              the shape (every call the observers make does);
 *                              LQ_ERR_NOT_IMPLEMENTED otherwise. */
int lq_sub_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream);
int lq_mul_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream);
int lq_div_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream);
int lq_maximum_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream);
int lq_minimum_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream);
int lq_round_f32(const float* x, float* out, size_t n, lq_stream stream);
int lq_clip_f32(const float* x, float* out, size_t n, double min_v, double max_v, lq_stream stream);
int lq_astype(const void* src, int src_dtype, void* dst, int dst_dtype, size_t n, lq_stream stream);
int lq_broadcast_f32(const float* src, float* out, size_t outer, size_t C, size_t inner, lq_stream stream);
int lq_reduce_minmax(const float* x, const int64_t* shape, int ndim, const int* axes, int n_axes, float* mn,
                     float* mx, lq_stream stream);

/* Eval-mode BatchNorm forward on (B, C, spatial) float32 (1-d / 2-d / 3-d alike):
 *     rstd[c] = 1 / float(sqrt(double(var[c]) + eps))
 *     y       = gamma[c] * (x - mean[c]) * rstd[c] + beta[c]        (float32, in that order)
 * IBackend::batch_norm_eval_forward (CpuBackend.h:9163-9208), what F.batch_norm runs when
 * not training (lucid/nn/functional/normalization.py:104-109).  gamma / beta NULL = 1 / 0.
 * It lets an un-fused conv + BN model run on the device, e.g. to check fuse_modules
 * against it (lucid/test/unit/quantization/test_static_ptq.py:90-99). */
int lq_batchnorm_eval_f32(const float* x, float* out, size_t B, int C, size_t spatial, const float* mean,
                          const float* var, const float* gamma, const float* beta, double eps, lq_stream stream);

/* ------------------------------------------------------------ quantize family */
/* min and max over everything but the channel axis, NaN-propagating.
 * Replaces reduce_min/reduce_max (IBackend.h:689-692; CpuBackend.h:12012,
 * Reduce.cpp:87-125) as used by MinMaxObserver / PerChannelMinMaxObserver
 * (lucid/quantization/observer.py:363-375,634-653) and nnqd.Linear
 * (lucid/nn/quantized/dynamic/linear.py:87-89).  mn, mx: device f32[C]. */
int lq_minmax(const float* x, size_t outer, size_t C, size_t inner, float* mn, float* mx,
              lq_stream stream);

/* lq_minmax for callers that cannot allocate (code under HIP graph capture, serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in Lucid.  Same
 * arguments, same results bit for bit; the partial results of the two-stage
 * reduction live in a 1 MiB array that is part of the library's device image
 * (one copy per GPU, held until the process ends), and the call makes no
 * hipMalloc / hipFree.  Limit: a reduction over short runs (inner < 64, C > 1)
 * needs 8 * C * inner bytes of partials and is refused with LQ_ERR_SHAPE beyond
 * 1 MiB (C * inner > 131072); every other shape fits (fewer slices per channel
 * are used when the usual number would not).  Nothing in the array has to be
 * cleared between calls: every partial that is read has been written by the same
 * call.  All calls on one GPU share the array, so calls that overlap on one GPU
 * (different streams, or one stream and a graph replay on another) race.
 * lq_init resolves the array's address for its device; without it the first call
 * on a device does. */
int lq_minmax_noalloc(const float* x, size_t outer, size_t C, size_t inner, float* mn, float* mx,
                      lq_stream stream);

/* calculate_qparams (lucid/quantization/_qparams.py:190-215) over C channels,
 * entirely on the device.  scale, zp: device f32[C]. */
int lq_calc_qparams(const float* mn, const float* mx, size_t C, int symmetric, int qmin, int qmax,
                    int is_signed, float eps, float* scale, float* zp, lq_stream stream);

/* quantize (lucid/quantization/_functional.py:164-182):
 *   code = clip(rint(x / s) + z, qmin, qmax), stored as q_dtype (LQ_I8 or
 *   LQ_I16) after adding code_offset (0 = Lucid's storage; -128 keeps a quint8
 *   code in an int8 for the signed MFMA operand).
 * scale, zp: f32[C]; device memory, or host memory when qparams_on_host != 0
 * (C must be 1 then: Lucid's Python-float scale). */
int lq_quantize(const float* x, void* q, int q_dtype, int code_offset, size_t outer, size_t C,
                size_t inner, const float* scale, const float* zp, int qparams_on_host, int qmin,
                int qmax, lq_stream stream);

/* dequantize (_functional.py:269-281): out = (f32(code) - z) * s. */
int lq_dequantize(const void* q, int q_dtype, int code_offset, float* out, size_t outer, size_t C,
                  size_t inner, const float* scale, const float* zp, int qparams_on_host,
                  lq_stream stream);

/* fake_quantize forward (_functional.py:299-313): (clip(rint(x/s)+z) - z) * s. */
int lq_fake_quantize(const float* x, float* out, size_t outer, size_t C, size_t inner,
                     const float* scale, const float* zp, int qparams_on_host, int qmin, int qmax,
                     lq_stream stream);

/* ------------------------------------------------------- elementwise members */
/* ReLU on float32 (IBackend::relu; CpuBackend vrelu_f32, Vdsp.cpp:130-133):
 * the activation between dynamic-quantized layers, whose outputs are float. */
int lq_relu_f32(const float* x, float* out, size_t n, lq_stream stream);

/* Observer state update: out_min = minimum(run_min, cur_min), out_max =
 * maximum(run_max, cur_max) over C channels (observer.py:370-371,652-653;
 * IBackend::minimum/maximum, CpuBackend.h:828-864).  run_* may be the scalar
 * +-inf seed broadcast over C (run_is_scalar != 0).  out_* may alias cur_*. */
int lq_minmax_fold(const float* run_min, const float* run_max, const float* cur_min,
                   const float* cur_max, size_t C, int run_is_scalar, float* out_min,
                   float* out_max, lq_stream stream);

/* Moving-average observers (lucid/quantization/observer.py:490-506 per tensor,
 * :1000-1018 per channel): out = seed ? cur : run + c * (cur - run) in float32.
 * Per tensor the seed test is isinf(run_min) elementwise; per channel everything is
 * seeded when every running minimum is still infinite.  run_* hold one value when
 * run_is_scalar (the +-inf start), else C. */
int lq_minmax_ema(const float* run_min, const float* run_max, const float* cur_min, const float* cur_max,
                  size_t C, int run_is_scalar, int per_channel, float averaging_constant, float* out_min,
                  float* out_max, lq_stream stream);

/* lucid.histc (IBackend::histogram_forward, CpuBackend.h:13276-13316) on float32
 * input: `bins` equal-width buckets over [lo, hi], the bucket taken in double
 * arithmetic as (int64)((v - lo) / ((hi - lo) / bins)), the right edge folded into
 * the last bucket, values outside skipped; float32 counts out (HistogramObserver's
 * running histogram, observer.py:819-838). */
int lq_histc_f32(const float* x, size_t n, double lo, double hi, int bins, float* out, lq_stream stream);

/* QFunctional.add / add_relu on codes (nn/quantized/functional_module.py:216-230):
 * out = quantize(relu?((qa - za)*sa + (qb - zb)*sb)) with every qparam a device
 * scalar.  Codes are int8 as stored (code + offset). */
int lq_add_requant_i8(const int8_t* qa, int a_offset, const float* a_scale, const float* a_zp,
                      const int8_t* qb, int b_offset, const float* b_scale, const float* b_zp,
                      size_t n, int relu, const float* out_scale, const float* out_zp, int out_qmin,
                      int out_qmax, int out_offset, int8_t* out, lq_stream stream);

/* F.adaptive_avg_pool2d(x, 1) on NHWC codes -> float32 [B, C]: Lucid pools the
 * float-carried values, so the result leaves the grid (it feeds the float input
 * of the classifier).  Exact integer sum of codes, then float32 scaling. */
int lq_global_avgpool_nhwc_i8(const int8_t* q, int code_offset, int B, int H, int W, int C,
                              const float* scale, const float* zp, float* out, lq_stream stream);

/* ------------------------------------------------- group-wise weight-only path */
/* engine.quantized.{quantize, dequantize, quantized_matmul}
 * (lucid/_C/bindings/bind_quantized.cpp:18-25; lucid/_C/ops/quantized/QuantizedMatmul.cpp:47-115;
 * lucid/quantization/_qgemm.py:69-320), which Lucid implements by calling MLX.  MLX is
 * not part of the Lucid checkout; these follow the documented contract
 * (_qgemm.py:84-97,167-171): per row and per group of group_size (32 / 64 / 128)
 * consecutive elements, s = (max - min) / (2^bits - 1), beta = min,
 * c = clip(round((w - beta) / s), 0, 2^bits - 1), w ~ c * s + beta; bits is 4 or 8;
 * codes are packed little-endian into 32-bit words (code j at bits [j*bits, (j+1)*bits)):
 * packed is [N, K*bits/32], scales and biases [N, K/group_size].  Decoding takes scales
 * and biases as given, so weights packed elsewhere under this contract load unchanged.
 * lq_wq_matmul: out[M,N] = x[M,K] . w_hat^T in float32 (transpose = True of
 * _qgemm.quantized_matmul).  M = 1 streams the packed weight through a dot-product kernel;
 * 2 <= M <= 64 (K a multiple of 512 / bits) runs on the matrix cores with the codes as one
 * bfloat16 operand and x split exactly into three bfloat16 parts, per-group sums scaled in
 * float32, partial sums of the k ranges added in a fixed order (results are reproducible);
 * larger M decodes into the workspace and runs the float32 GEMM. */
int lq_wq_quantize(const float* w, int N, int K, int group_size, int bits, uint32_t* packed, float* scales,
                   float* biases, lq_stream stream);
int lq_wq_dequantize(const uint32_t* packed, const float* scales, const float* biases, int N, int K, int group_size,
                     int bits, float* out, lq_stream stream);
int lq_wq_matmul(const float* x, const uint32_t* packed, const float* scales, const float* biases, int M, int N, int K,
                 int group_size, int bits, float* out, lq_stream stream);

/* y[m,n] = act(y[m,n] + bias[n]) in place on float32 [M,N]; bias may be NULL, act is
 * ReLU when relu != 0: the float bias / fused ReLU after the weight-only matmul
 * (lucid/nn/quantized/mlx_linear.py forward). */
int lq_bias_act_f32(float* y, const float* bias, size_t M, int N, int relu, lq_stream stream);

/* ------------------------------------------------- ranges kept by the producer */
/* Dynamic per-tensor quantization of a small tensor (n <= 262144) in one launch:
 * global min / max (MinMaxObserver, observer.py:363-375; x.min() / x.max() in
 * nnqd.Linear, dynamic/linear.py:87-89), calculate_qparams (_qparams.py:198-215)
 * and quantize (_functional.py:164-182) - the results of lq_minmax +
 * lq_calc_qparams + lq_quantize bit for bit.  scale, zp: one float each (device);
 * mn_out, mx_out optional.  Larger tensors: LQ_ERR_NOT_IMPLEMENTED (use the
 * three calls, which are bandwidth-bound there). */
int lq_quantize_tensor_dynamic_i8(const float* x, size_t n, int symmetric, int qmin, int qmax, int is_signed,
                                  float eps, int code_offset, float* scale, float* zp, float* mn_out,
                                  float* mx_out, int8_t* q, lq_stream stream);

/* A dynamic-quantized Linear on a small activation in ONE launch: nnqd.Linear.forward
 * (lucid/nn/quantized/dynamic/linear.py:87-99) for x [M, K] float32 with M <= 64,
 * K % 16 == 0, K <= 6080 (16 rows of codes stay in LDS) and M * K <= 65536 - the tensor's
 * min / max, calculate_qparams, the activation codes (kept in LDS), the integer GEMM against w [N, K] int8 codes with
 * per-row scales w_scale [N] and code sums wsum [N], float32 bias [N] or NULL, optional
 * ReLU; out [M, N] float32.  The bits of lq_quantize_tensor_dynamic_i8 followed by
 * lq_qlinear_i8 (mode F32).  Symmetric weights only.  Anything else:
 * LQ_ERR_NOT_IMPLEMENTED (use the two calls). */
int lq_dynamic_linear_small_f32(const float* x, int M, int K, const int8_t* w, int N, const float* w_scale,
                                const int32_t* wsum, const float* bias, int relu, int symmetric, int qmin, int qmax,
                                int is_signed, float eps, int code_offset, float* out, lq_stream stream);

/* Two dynamic-quantized Linears in ONE launch: y = L2(act1(L1(x))) with each layer as
 * lq_dynamic_linear_small_f32 computes it (the hidden activation's min / max, qparams and codes
 * included: the blocks of layer 1 pass their tiles and ranges through the stream's scratch and
 * the last of them to arrive runs layer 2) and relu1 / relu2 the optional ReLU behind each.  x [M, K1] float32, w1 [N1, K1], w2 [N2, N1] int8 codes with their
 * per-row scales, code sums and float32 biases (or NULL); out [M, N2] float32.  M <= 64,
 * K1 % 16 == 0 and <= 1024, N1 % 16 == 0 and <= 256, N2 <= 64; anything else
 * LQ_ERR_NOT_IMPLEMENTED.  Same bits as the separate calls (Linear, ReLU, Linear of a
 * quantize_dynamic'd MLP: lucid/nn/quantized/dynamic/linear.py:84-99).  No counterpart in Lucid. */
int lq_dynamic_mlp2_small_f32(const float* x, int M, int K1, const int8_t* w1, int N1, const float* w1_scale,
                              const int32_t* w1sum, const float* bias1, int relu1, const int8_t* w2, int N2,
                              const float* w2_scale, const int32_t* w2sum, const float* bias2, int relu2, int symmetric,
                              int qmin, int qmax, int is_signed, float eps, int code_offset, float* out,
                              lq_stream stream);

/* Dynamic per-row quantization in one pass: for every row of x [rows, cols],
 * min / max of the row (PerChannelMinMaxObserver with ch_axis = 0,
 * observer.py:634-653), its qparams (calculate_qparams, _qparams.py:198-215) and
 * its int8 codes (quantize, _functional.py:164-182) - the results of lq_minmax +
 * lq_calc_qparams + lq_quantize bit for bit, with x read once.  This is the
 * per-token activation quantization in front of an LLM-shaped Linear.  scale,
 * zp: [rows] out; mn_out, mx_out: optional [rows] out.  cols must be a multiple
 * of 4, at most 16384, x 16-byte aligned (LQ_ERR_NOT_IMPLEMENTED otherwise: use
 * the three calls). */
int lq_quantize_rows_dynamic_i8(const float* x, size_t rows, size_t cols, int symmetric, int qmin, int qmax,
                                int is_signed, float eps, int code_offset, float* scale, float* zp,
                                float* mn_out, float* mx_out, int8_t* q, lq_stream stream);

/* nnqd.Linear takes x.min() / x.max() of its input on every forward
 * (lucid/nn/quantized/dynamic/linear.py:87-89): a full pass over a tensor some
 * kernel has just written.  The float32 kernels below can keep that range as a
 * by-product: pass them a device buffer of lq_range_buffer_bytes() bytes (no
 * initialisation needed) and every block stores the min / max of what it wrote
 * into a slot of its own.  lq_calc_qparams_from_range reduces the slots and is
 * then calculate_qparams(min, max) (_qparams.py:190-215), bit-identical to
 * lq_minmax + lq_calc_qparams; mn_out / mx_out (optional) receive the range. */
size_t lq_range_buffer_bytes(void);
int lq_calc_qparams_from_range(const float* range, int symmetric, int qmin, int qmax, int is_signed,
                               float eps, float* scale, float* zp, float* mn_out, float* mx_out,
                               lq_stream stream);

/* ------------------------------------------------- float32 steps of a ViT block */
/* What Lucid's dynamic-quantized ViT keeps in float32 between its int8 Linears
 * (lucid/models/vision/vit/_model.py:132-161,202-204,275-278,449-458).  Tolerance
 * parity (1e-4 relative against a float32 CPU evaluation): summation orders differ.
 * range, where present, may be null. */

/* LayerNorm over the last axis of [rows, cols] (IBackend::layer_norm_forward;
 * lucid/_C/backend/cpu/Norm.cpp:35-65: mean, centred dot product / N,
 * rstd = 1/sqrt(var + eps), (c * rstd) * gamma + beta). */
int lq_layernorm_f32(const float* x, const float* gamma, const float* beta, float* out, long rows, int cols,
                     float eps, float* range, lq_stream stream);

/* LayerNorm in front of a dynamic-quantized Linear without the float32 round trip
 * (nn.LayerNorm followed by nnqd.Linear: Norm.cpp:35-65, then dynamic/linear.py:87-92).
 * lq_layernorm_stats_f32 writes each row's mean and rstd to stats [rows, 2] and keeps
 * the min / max of the normalized values in `range` (lq_range_buffer_bytes() bytes);
 * after lq_calc_qparams_from_range, lq_layernorm_quantize_i8 normalizes again with
 * those statistics and writes the int8 codes - bit for bit the codes of
 * lq_layernorm_f32 + lq_quantize.  Rows must be a multiple of 4 floats, at most
 * 2048, 16-byte aligned (LQ_ERR_NOT_IMPLEMENTED otherwise). */
int lq_layernorm_stats_f32(const float* x, const float* gamma, const float* beta, long rows, int cols, float eps,
                           float* stats, float* range, lq_stream stream);
int lq_layernorm_quantize_i8(const float* x, const float* gamma, const float* beta, const float* stats, long rows,
                             int cols, const float* scale, const float* zp, int qmin, int qmax, int code_offset,
                             int8_t* q, lq_stream stream);

/* GELU, exact erf form (lucid/nn/functional/activations.py:219, approximate="none"). */
int lq_gelu_f32(const float* x, float* out, size_t n, float* range, lq_stream stream);

/* out = a + b (IBackend::add on float32; the residual joins). */
int lq_add_f32(const float* a, const float* b, float* out, size_t n, lq_stream stream);

/* Scaled dot-product attention (IBackend::sdpa_forward, CpuBackend.h:7603-7730:
 * softmax(scale * Q K^T) V, no mask, no dropout) read straight from the packed
 * activation of the qkv Linear, [B, T, 3, H, D] (vit/_model.py:137-141), writing
 * [B, T, H*D] (vit/_model.py:158).  D must be 64 and T <= 208 (ViT-B/16: T = 197);
 * anything else returns LQ_ERR_NOT_IMPLEMENTED. */
int lq_attention_f32(const float* qkv, float* out, int B, int T, int H, int D, float scale,
                     float* range, lq_stream stream);

/* Patch embedding, a convolution whose stride equals its kernel
 * (vit/_model.py:62-69), as im2col + GEMM: image [B,C,H,W] -> rows
 * [B*(H/p)*(W/p), C*p*p] in (c, ph, pw) column order - the order of the conv
 * weight [dim, C, p, p] flattened. */
int lq_patchify_f32(const float* img, float* out, int B, int C, int H, int W, int patch, lq_stream stream);

/* Float32 convolution of an NCHW image with an OIHW filter, zero padding (pad_h / pad_w
 * on both sides), as im2col + GEMM (IBackend::conv_nd_forward, CpuBackend.h:8124-8257;
 * Im2Col.cpp:59-100; output size ConvNd.cpp:56-59).  It is what a calibration pass
 * through a prepared convolutional model and the forward of a QAT convolution run on;
 * inference goes through lq_qconv2d_i8.  out: [B, Cout, OH, OW].  Synchronises the
 * stream before it returns (its scratch comes from lq_alloc). */
int lq_conv2d_f32(const float* x, const float* w, const float* bias, float* out, int B, int Cin, int H, int W, int Cout,
                  int KH, int KW, int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, int groups,
                  lq_stream stream);

/* out[M,N] = a[M,K] . w[N,K]^T + bias[N] in float32 (IBackend::linear, CpuBackend.h:4525);
 * bias may be null.  Products are formed from three-way bfloat16 splits of both operands
 * (six part products, float32 accumulation): 2^-24 relative accuracy per product, as a
 * float32 multiply-add, at the rate of the bfloat16 matrix instruction. */
int lq_sgemm_nt_f32(const float* a, const float* w, const float* bias, float* out, int M, int N, int K,
                    lq_stream stream);

/* dst[r, 0:cols] = src[r * src_row_stride + 0:cols]: strided row gather (class-token
 * pooling x[:, 0], vit/_model.py `_pool`). */
int lq_gather_rows_f32(const float* src, size_t src_row_stride, float* dst, size_t rows, size_t cols,
                       lq_stream stream);

/* tokens[b,0,:] = cls + pos[0], tokens[b,1+i,:] = patches[b,i,:] + pos[1+i]
 * (cat + position table, vit/_model.py:452-454); out is [B, T, D], patches [B, T-1, D]. */
int lq_assemble_tokens_f32(const float* patches, const float* cls, const float* pos, float* out, int B, int T,
                           int D, lq_stream stream);

/* lq_patchify_f32, lq_sgemm_nt_f32 and lq_assemble_tokens_f32 in one launch, with the same
 * arithmetic in the same order (vit/_model.py:62-69 and 452-454): the GEMM reads its rows
 * straight from the image [B,C,H,W], adds bias[D] and then the position row, and writes
 * token rows out[B, 1 + (H/p)*(W/p), D]; row 0 of every image is cls + pos[0].
 * w: [D, C*p*p], cls: [D], pos: [1 + (H/p)*(W/p), D].  bias may be null. */
int lq_patch_embed_f32(const float* img, const float* w, const float* bias, const float* cls, const float* pos,
                       float* out, int B, int C, int H, int W, int patch, int D, lq_stream stream);

/* The other merges of QFunctional (functional_module.py:220-246) on codes:
 * fq(act(x OP y)), OP = add (0) or mul (1), y a second code tensor or - when qb is
 * NULL - the float scalar (add_scalar / mul_scalar).  Each operand is dequantized
 * with its own float32 steps, OP and the optional ReLU are float32, then the usual
 * requantize. */
int lq_binary_requant_i8(int op, const int8_t* qa, int a_offset, const float* a_scale, const float* a_zp,
                         const int8_t* qb, int b_offset, const float* b_scale, const float* b_zp, float scalar,
                         size_t n, int relu, const float* out_scale, const float* out_zp, int out_qmin,
                         int out_qmax, int out_offset, int8_t* out, lq_stream stream);

/* One operand of QFunctional.cat (functional_module.py:232-234): codes [rows, cols]
 * on their own grid re-expressed on the output grid, written with row stride out_ld
 * into the operand's column slot of the concatenated tensor. */
int lq_requant_rows_i8(const int8_t* q, int q_offset, const float* scale, const float* zp, size_t rows,
                       size_t cols, int8_t* out, size_t out_ld, const float* out_scale, const float* out_zp,
                       int out_qmin, int out_qmax, int out_offset, lq_stream stream);

/* Quantized Linear on a float activation that lies on no grid - literally
 * lucid/nn/quantized/linear.py:199-215: dequantize(weight) -> x @ W^T + bias ->
 * [relu] -> [fake_quantize].  float32 accumulation; for small layers (e.g. the
 * classifier after global pooling), not a throughput path. */
int lq_qlinear_w8a32(const float* x, const int8_t* w, const float* w_scale, const float* w_zp,
                     const float* bias, int M, int N, int K, int relu, int fake_quantize_out,
                     const float* out_scale, const float* out_zp, int out_qmin, int out_qmax,
                     float* out, lq_stream stream);

/* ------------------------------------------------------- quantized Linear */
/* Output forms of the fused GEMM epilogue. */
#define LQ_OUT_ACC_I32 0       /* raw int32 accumulators                         */
#define LQ_OUT_F32 1           /* dequantized float32 (nnqd.Linear's result)     */
#define LQ_OUT_F16 2           /* dequantized float16, RNE (core/Half.h:80-110)  */
#define LQ_OUT_REQUANT_I8 3    /* code on the output grid, stored + out_offset   */
#define LQ_OUT_FAKEQUANT_F32 4 /* float-carried value on the output grid         */

/* sum_k w[n,k] for every weight row: the zero-point correction term, computed
 * once when a module is converted (from_float, lucid/nn/quantized/linear.py:217-236). */
int lq_rowsum_i8(const int8_t* w, int32_t* out, int N, int K, lq_stream stream);

/* Quantized Linear forward.  Replaces the composite that
 * lucid/nn/quantized/linear.py:199-215 (static), intrinsic.py:131-133 (fused
 * ReLU) and dynamic/linear.py:84-99 (dynamic) build from dequantize +
 * IBackend::linear (IBackend.h:960-966; CpuBackend.h:4525-4569) +
 * fake_quantize, by its exact integer identity:
 *     acc[m,n] = sum_k a[m,k] * w[n,k]                              (int32)
 *     y = f32(acc - a_zp*wsum[n]) * (a_scale[m|0] * w_scale[n]) + bias[n]
 *     y = relu(y) if relu,  y = gelu(y) if gelu
 *     y = y + residual[m,n] if residual
 *     out = per out_mode
 * a: int8 [M,K] activation codes as stored (a quint8 code c is stored as
 * c - 128, and a_zp is then Z - 128); w: int8 [N,K].  All pointers are device
 * pointers; scales and output qparams are read on the device so no host
 * synchronisation is needed between layers. */
/* Optional residual join on codes, fused into the REQUANT_I8 epilogue: what
 * QFunctional.add / add_relu (lucid/nn/quantized/functional_module.py:224-230) does to
 * this layer's output and a second activation, without the layer's own output ever
 * reaching memory.  With c1 the layer's code on (out_scale, out_zp):
 *     x1 = (c1 - out_zp) * out_scale          x2 = (q[m,n] - offset - zp) * scale
 *     y  = x1 + x2,  y = max(y, 0) if relu
 *     out[m,n] = code of y on (out_scale', out_zp', [out_qmin', out_qmax']) + out_offset'
 * (primed = the fields of this struct), bit for bit what lq_add_requant_i8 gives on
 * the stored intermediate.  q == NULL: no join. */
typedef struct {
    const int8_t* q;        /* [M, ld] stored codes of the other operand          */
    long ld;                /* row stride in elements; 0 means N (Cout)           */
    int offset;             /* storage offset of q's codes                        */
    const float* scale;     /* [1] grid of q                                      */
    const float* zp;        /* [1]                                                */
    int relu;
    const float* out_scale; /* [1] grid of the joined result                      */
    const float* out_zp;    /* [1]                                                */
    int out_qmin, out_qmax, out_offset;
} lq_join_args;

typedef struct {
    const int8_t* a;
    const int8_t* w;
    int M, N, K;
    const int32_t* wsum;   /* [N], required when a_zp != 0                   */
    int a_zp;              /* zero point of the stored codes (host value)       */
    const float* a_zp_dev; /* optional device scalar (a zero point computed on the
                              device, as in nnqd.Linear): the effective zero
                              point is (int)*a_zp_dev + a_zp                    */
    const float* a_scale;  /* [M] when a_scale_per_row, else [1]             */
    int a_scale_per_row;
    const float* w_scale;  /* [N]                                            */
    const void* bias;      /* [N] or NULL                                    */
    int bias_dtype;        /* LQ_F32 or LQ_F16                               */
    int relu;
    int out_mode;          /* LQ_OUT_*                                       */
    const float* out_scale;/* [1], modes REQUANT_I8 / FAKEQUANT_F32          */
    const float* out_zp;   /* [1]                                            */
    int out_qmin, out_qmax, out_offset;
    void* out;             /* [M, ldo] in the type out_mode implies          */
    long ldo;              /* output row stride in elements; 0 means N       */
    int force_path;        /* 0 = choose; 1 = tile, 2 = skinny, 3 = naive    */
    int tile_config;       /* tuning: low byte 0 = choose, 1..12 = a tile shape of the
                              four-wavefront kernel, 13 / 14 / 16 / 21 / 22 = 256x352 /
                              256x256 / 256x192 / 224x192 / 160x256 tiles of the
                              eight-wavefront kernel (plain GEMM, K % 64 == 0), 17 = 256x352 tiles with one wavefront per SIMD
                              (plain GEMM, K % 128 == 0, K >= 256, float16 output or raw
                              accumulators; never chosen automatically),
                              15 / 18 / 19 (convolutions only) = one block per box of
                              256 / 128 / 64 output positions x 64 channels with the box's
                              input halo held in LDS (stride 1, Cin/groups % 64 == 0, no
                              join), 20 (the packed route of a convolution with at most four
                              input channels, filter row of at most 256 bytes, no join) =
                              boxes of 16 x 16 output positions x 64 channels with the
                              filter in registers and the box's input halo in LDS;
                              next byte 0 = choose, 1 = one block per tile,
                              2 = stream-K work split, 3 = stream-K over the
                              leftover tiles of the last round only; bits 16..30
                              = number of leading 256-column tiles computed with
                              256x256 tiles, the remaining columns as a problem of
                              their own (0 = no split)                          */
    const float* residual; /* optional float32 [M, ldr] added after the activation:
                              out = act(y) + residual (x + linear(...), the
                              residual joins of a transformer block,
                              vit/_model.py:276-277); modes F32 / F16 only        */
    long ldr;              /* residual row stride in elements; 0 means N     */
    lq_join_args join;     /* optional join on codes; mode REQUANT_I8 only   */
    int gelu;              /* mode F32: exact-erf GELU
                              (lucid/nn/functional/activations.py:219) applied to
                              y after the bias / ReLU and before a residual - the
                              fc1 -> GELU of a transformer MLP in one kernel   */
    float* range;          /* optional range buffer (lq_range_buffer_bytes()) that
                              receives the min / max of the stored output, for
                              lq_calc_qparams_from_range of the next dynamic
                              quantizer; mode F32, tile kernel only             */
    const int32_t* w_zp;   /* optional [N] zero points of the weight rows, as stored
                              codes (device): per-channel affine weights
                              (lucid/quantization/_qscheme.py per_channel_affine, kept by
                              from_float, lucid/nn/quantized/linear.py:217-236).  The
                              effective accumulator is then
                                sum_k (a[m,k] - a_zp) * (w[n,k] - w_zp[n])
                                = acc - a_zp*wsum[n] - w_zp[n]*sum_k a[m,k] + K*a_zp*w_zp[n],
                              exact in int32 (K <= 33025); the row sums of a are taken by
                              the call, wsum is required.  NULL = symmetric weights;
                              LQ_ERR_VALUE with mode ACC_I32 (the raw sums a * w);
                              not with range.                                      */
} lq_qlinear_args;

int lq_qlinear_i8(const lq_qlinear_args* args, lq_stream stream);

/* The tile_config (same encoding as the field above) that the calling thread's last
 * tile-kernel launch resolved to - what the autotuner chose when 0 was passed.  For
 * benchmarks and tests; 0 before the first such launch.  No counterpart in Lucid. */
int lq_last_tile_config(void);

/* The tuner's choices as text, so that a deployment tunes once: one line per problem shape
 * ("lq-tune-1", the shape key's integers, the chosen tile_config).  lq_tune_export writes what
 * this process has chosen so far into buf (NUL-terminated); *needed receives the bytes
 * required, and buf may be NULL to ask for that alone.  lq_tune_import adds the lines of
 * `text` to the table (later launches of those shapes skip the timing; lines that do not
 * start with "lq-tune-1" are skipped, a malformed one is LQ_ERR_VALUE); *accepted (may be
 * NULL) receives the number of entries taken.  A file of such lines named by the environment
 * variable LQ_TUNE_FILE is imported before the first lookup.  Results do not depend on the
 * tile shape, only the time does.  No counterpart in Lucid. */
int lq_tune_export(char* buf, size_t capacity, size_t* needed);
int lq_tune_import(const char* text, int* accepted);

/* The same forward launched n times back to back from native code: for
 * launch-bound callers (decode-shaped layers run for ~10 us, less than an
 * interpreter's call overhead) and for timing.  No counterpart in Lucid. */
int lq_qlinear_i8_n(const lq_qlinear_args* args, int n, lq_stream stream);

/* ------------------------------------------------------- quantized Conv2d */
/* Quantized Conv2d forward.  Replaces the composite of
 * lucid/nn/quantized/conv.py:168-184 (+ intrinsic.py:334-336 for the fused
 * ReLU): dequantize kernel -> IBackend::conv_nd_forward (IBackend.h:1469-1482;
 * per-image im2col + sgemm, CpuBackend.h:8124-8257) -> per-channel bias ->
 * fake_quantize, by the same integer identity as lq_qlinear_i8 with
 *     m = (b, oh, ow),  n = cout,  k = (kh, kw, cin_in_group).
 * Layouts differ from Lucid's NCHW / OIHW on purpose: activation codes are
 * NHWC [B,H,W,Cin] and weight codes [Cout,KH,KW,Cin/groups], so that k runs
 * over contiguous bytes (use lq_quantize_nchw_to_nhwc, lq_repack_oihw_to_ohwi_i8
 * and lq_dequantize_nhwc_to_nchw at the model boundary).  Zero padding of the
 * float image (Im2Col.cpp:59-100) becomes padding with the code a_zp.
 * Output: NHWC [B,OH,OW,Cout], OH/OW per lucid/_C/nn/ConvNd.cpp:56-59 with
 * separate low/high pads ("same" padding can be asymmetric,
 * lucid/nn/modules/conv.py:44-55). */
typedef struct {
    const int8_t* x;       /* NHWC codes as stored                           */
    const int8_t* w;       /* [Cout,KH,KW,Cin/groups] codes                  */
    int B, H, W, Cin, Cout, KH, KW;
    int stride_h, stride_w, pad_h_lo, pad_h_hi, pad_w_lo, pad_w_hi, dil_h, dil_w, groups;
    const int32_t* wsum;   /* [Cout] sum of each filter's codes              */
    int a_zp;              /* zero point of the stored codes; also the pad code */
    const float* a_scale;  /* [1]                                            */
    const float* w_scale;  /* [Cout]                                         */
    const void* bias;      /* [Cout] or NULL                                 */
    int bias_dtype;
    int relu;
    int out_mode;          /* LQ_OUT_*                                       */
    const float* out_scale;
    const float* out_zp;
    int out_qmin, out_qmax, out_offset;
    void* out;             /* NHWC [B,OH,OW,Cout]                            */
    int force_path;        /* 0 = choose; 1 = gemm (1x1), 2 = implicit GEMM,
                              3 = explicit im2col + GEMM, 4 = naive,
                              5 = packed 4-channel image (Cin <= 4),
                              6 = the same with x and w already packed
                              (lq_quantize_nchw_to_packed4, lq_pack4_filter_i8)  */
    int tile_config;
    lq_join_args join;     /* optional join on codes (NHWC, ld = Cout): the residual
                              add of a bottleneck block fused into its last
                              convolution; mode REQUANT_I8 only                  */
    const int32_t* w_zp;   /* optional [Cout] zero points of the filters' stored codes
                              (device), as lq_qlinear_args.w_zp; the window sums of the
                              image come from a convolution with an all-ones filter, so
                              taps in the padding count as a_zp and cancel exactly.
                              NULL = symmetric; LQ_ERR_VALUE with mode ACC_I32     */
} lq_qconv2d_args;

int lq_qconv2d_i8(const lq_qconv2d_args* args, lq_stream stream);

/* Model-boundary layout helpers (per-tensor qparams as device scalars):
 * quantize float32 NCHW into int8 NHWC codes; the inverse float view; and the
 * one-time repack of weight codes from Lucid's OIHW buffer. */
int lq_quantize_nchw_to_nhwc(const float* x, int8_t* q, int code_offset, int B, int C, int H, int W,
                             const float* scale, const float* zp, int qmin, int qmax,
                             lq_stream stream);
int lq_dequantize_nhwc_to_nchw(const int8_t* q, int code_offset, float* out, int B, int C, int H,
                               int W, const float* scale, const float* zp, lq_stream stream);

/* A first layer with at most four input channels (the RGB stem of a vision model,
 * lucid/nn/quantized/modules.py:266-292 followed by conv.py:168-184) without the NHWC code
 * tensor in between: lq_quantize_nchw_to_packed4 quantizes the float32 NCHW image straight
 * into the four-channel, spatially pre-padded code image that the few-channel route of
 * lq_qconv2d_i8 gathers from (padding and spare channels hold fill_code, the zero-point
 * code as stored; extents from lq_qconv2d_packed4_geometry), lq_pack4_filter_i8 lays the
 * filter codes out to match once ([Cout,KH,KW,Cin] -> [Cout,KH,KWp,4], zeros in the added
 * taps and channels), and lq_qconv2d_i8 with force_path = 6 takes both as x and w (H, W,
 * pads, KW, Cin still describe the logical layer).  Same codes as lq_quantize_nchw_to_nhwc
 * + force_path 5. */
int lq_qconv2d_packed4_geometry(const lq_qconv2d_args* args, int* Hp, int* Wp, int* KWp);
int lq_quantize_nchw_to_packed4(const float* x, int8_t* out, int code_offset, int B, int C, int H, int W,
                                int pad_h_lo, int pad_w_lo, int Hp, int Wp, const float* scale, const float* zp,
                                int qmin, int qmax, int fill_code, lq_stream stream);
int lq_pack4_filter_i8(const int8_t* w, int8_t* out, int Cout, int KH, int KW, int Cin, lq_stream stream);
int lq_repack_oihw_to_ohwi_i8(const int8_t* w, int8_t* out, int O, int I, int KH, int KW,
                              lq_stream stream);

/* Quantized Conv3d forward as an implicit GEMM (lucid/nn/quantized/conv.py:545-700:
 * dequantize kernel -> F.conv3d -> bias -> fake_quantize; IBackend::conv_nd_forward,
 * IBackend.h:1469-1482, with three spatial dims), by the integer identity of
 * lq_qconv2d_i8 with
 *     m = (b, od, oh, ow),  n = cout,  k = (kd, kh, kw, cin_in_group).
 * Activation codes are channels-last NDHWC [B,D,H,W,Cin], weight codes
 * [Cout,KD,KH,KW,Cin/groups] (lq_transpose_i8 and lq_repack_oihw_to_ohwi_i8 with
 * KH*KW := KD*KH*KW make them from Lucid's layouts); the taps are gathered by the
 * GEMM's tile loader, so no patch matrix is written.  Zero padding becomes padding
 * with the code a_zp; groups run in one launch.  stride / pad_lo / pad_hi /
 * dilation are (depth, height, width).  Output: NDHWC [B,OD,OH,OW,Cout].
 * Needs Cin/groups % 16 == 0 and 16-byte aligned tensors (LQ_ERR_NOT_IMPLEMENTED
 * otherwise: use the explicit route below). */
typedef struct {
    const int8_t* x;       /* NDHWC codes as stored                          */
    const int8_t* w;       /* [Cout,KD,KH,KW,Cin/groups] codes               */
    int B, D, H, W, Cin, Cout, KD, KH, KW;
    int stride[3], pad_lo[3], pad_hi[3], dilation[3], groups;
    const int32_t* wsum;   /* [Cout] sum of each filter's codes              */
    int a_zp;              /* zero point of the stored codes; also the pad code */
    const float* a_scale;  /* [1]                                            */
    const float* w_scale;  /* [Cout]                                         */
    const void* bias;      /* [Cout] or NULL                                 */
    int bias_dtype;
    int relu;
    int out_mode;          /* LQ_OUT_*                                       */
    const float* out_scale;
    const float* out_zp;
    int out_qmin, out_qmax, out_offset;
    void* out;             /* NDHWC [B,OD,OH,OW,Cout]                        */
    int tile_config;       /* 0 = choose; shapes 3, 4, 5, 6, 9 have the gather, 15 is
                              the halo-in-LDS kernel (see lq_qlinear_args)       */
    const int32_t* w_zp;   /* optional [Cout] zero points of affine filters, as
                              lq_qconv2d_args.w_zp                            */
} lq_qconv3d_args;

int lq_qconv3d_i8(const lq_qconv3d_args* args, lq_stream stream);

/* Quantized Conv3d (lucid/nn/quantized/conv.py:545-700: dequantize kernel -> F.conv3d ->
 * bias -> fake_quantize) as an explicit GEMM on codes (any channel count; also what the
 * transposed convolution uses).  lq_transpose_i8 (batched byte
 * transpose: src[b] R x Cn -> dst[b] Cn x R, batches src_stride / dst_stride bytes
 * apart) turns Lucid's (B, C, D*H*W) codes channels-last; lq_im2col_ndhwc_i8 gathers the
 * taps of the channels [c0, c0 + Cg) of one group from (B, D, H, W, C) codes into
 * cols [B*OD*OH*OW, KD*KH*KW*Cg], k = ((kd*KH + kh)*KW + kw)*Cg + c, taps in the padding
 * reading pad_code (the input zero point's stored code); lq_qlinear_i8 multiplies it
 * with that group's kernel rows [Cout/groups, K] (the (O, I, KD*KH*KW) buffer turned by
 * lq_repack_oihw_to_ohwi_i8) with the usual fused epilogue; lq_transpose_i8 again writes
 * the [L, Cout/groups] result of each batch into its channel slice of the
 * (B, Cout, L) output.  insert > 1 reads the input as if insert - 1 zero-point codes
 * stood between neighbouring samples: the zero insertion of ConvTranspose3d
 * (lucid/nn/quantized/conv_transpose.py:484-640), which is then this stride-1
 * convolution with the flipped kernel.  kernel / stride / pad_lo / dilation / insert /
 * out_size are host arrays of three ints (depth, height, width). */
int lq_im2col_ndhwc_i8(const int8_t* x, int8_t* cols, int B, int D, int H, int W, int C, int c0, int Cg,
                       const int* kernel, const int* stride, const int* pad_lo, const int* dilation,
                       const int* insert, const int* out_size, int pad_code, lq_stream stream);
int lq_transpose_i8(const int8_t* src, int8_t* dst, int batches, size_t R, size_t Cn, size_t src_stride,
                    size_t dst_stride, lq_stream stream);

/* F.pad on the last two axes of a float32 tensor seen as `planes` images of H x W
 * (lucid/nn/modules/conv.py:104-123 pre-pads this way for padding_mode != "zeros"; mode 0
 * pads with zeros, for the uneven amounts of padding="same"): mode 1 reflect, 2 replicate,
 * 3 circular.  out is [planes, H+top+bottom, W+left+right].  The float-input form of the
 * quantized convolutions runs on it. */
int lq_pad_planes_f32(const float* x, float* out, size_t planes, int H, int W, int pad_top, int pad_bottom,
                      int pad_left, int pad_right, int mode, lq_stream stream);

/* F.pad with mode reflect (1) / replicate (2) / circular (3) on NHWC codes: how a
 * quantized convolution with padding_mode != "zeros" pads before convolving with
 * padding 0 (lucid/nn/modules/conv.py:104-123).  The padded float image is a gather
 * of the original, so the codes are gathered the same way; out is
 * [B, H+top+bottom, W+left+right, C]. */
int lq_pad_nhwc_i8(const int8_t* x, int8_t* out, int B, int H, int W, int C, int pad_top, int pad_bottom,
                   int pad_left, int pad_right, int mode, lq_stream stream);

/* Max-pool on NHWC codes (F.max_pool2d between quantized layers of a ResNet
 * stem): quantisation is monotone, so pooling codes equals pooling values. */
int lq_maxpool2d_nhwc_i8(const int8_t* x, int8_t* out, int B, int H, int W, int C, int KH, int KW,
                         int stride_h, int stride_w, int pad_h, int pad_w, lq_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* LUCID_HIP_H */
