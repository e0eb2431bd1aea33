/*
 * kxc_hip.h -- C ABI of libkxc_hip.so, the MI355X (gfx950) backend for the
 * kxc compiler's lowered-operator hot path.
 *
 * Plain C: pointers, sizes and POD structs only.  Every data pointer passed to
 * an operator is a DEVICE pointer (from kxc_hip_alloc or any other HIP
 * allocation); `stream` is a hipStream_t passed as void* (NULL = the calling
 * thread's current stream set with kxc_hip_set_stream, else the null stream).
 * Every entry point returns 0 on success and a non-zero code on failure; the
 * message is then available from kxc_hip_last_error() on the same thread.
 * Operators only enqueue work; they do not synchronise.
 *
 * Each declaration cites the reference interface (relative to the reference
 * checkout) that it implements on the GPU or that would bind it.
 */
#ifndef KXC_HIP_H_
#define KXC_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KXC_HIP_OK 0
#define KXC_HIP_ERR_INVALID 1      /* bad argument / unsupported shape */
#define KXC_HIP_ERR_RUNTIME 2      /* a HIP runtime call failed */
#define KXC_HIP_ERR_COMPILE 3      /* hipRTC compilation failed */
#define KXC_HIP_ERR_NO_DEVICE 4    /* no usable GPU */

/* Message of the last failure on the calling thread ("" if none). */
const char* kxc_hip_last_error(void);
/* ABI version of this library (bumped on incompatible changes). */
int32_t kxc_hip_abi_version(void);

/* ========================================================================
 * 1. Device API -- the calls a HIPDeviceAPI subclass of the reference's
 *    DeviceAPI (include/base/device_api.h:77-123) forwards to, one for one
 *    with CUDADeviceAPI (src/base/device/cuda_device_api.cc:75-328).
 * ===================================================================== */

/* DeviceAttributes (include/base/device_api.h:42-63) as a POD. */
typedef struct kxc_hip_device_attrs {
    int32_t exists;                      /* 0 when no device / no runtime; never an error */
    int32_t warp_size;                   /* 64 on gfx950 */
    int64_t max_threads_per_block;
    int64_t max_shared_memory_per_block; /* LDS bytes a workgroup may use */
    int64_t max_shared_memory_per_multiprocessor;
    int64_t multi_processor_count;       /* compute units */
    int64_t max_clock_rate_khz;
    int64_t max_registers_per_block;
    int64_t l2_cache_size_bytes;
    int64_t total_global_memory;
    int64_t available_global_memory;
    int64_t max_threads_per_multiprocessor;
    int32_t compute_version_major;
    int32_t compute_version_minor;
    int32_t api_version;
    int32_t driver_version;
    char device_name[128];
    char arch[32];                       /* "gfx950" */
    char status[128];                    /* reason text when exists == 0 */
} kxc_hip_device_attrs;

/* GetTargetKind (cuda_device_api.cc:218-221 returns "cuda"): returns "hip". */
const char* kxc_hip_target_kind(void);
/* Device enumeration (src/base/device_api.cc:344,395-402).  *count = 0 without a GPU. */
int32_t kxc_hip_device_count(int32_t* count);
/* GetDeviceAttributes (cuda_device_api.cc:159-216): never fails, exists = 0 + status text instead. */
int32_t kxc_hip_device_attributes(int32_t device_id, kxc_hip_device_attrs* out);
/* SetDevice (cuda_device_api.cc:77-88). */
int32_t kxc_hip_set_device(int32_t device_id);
/* AllocDataSpace / FreeDataSpace (cuda_device_api.cc:90-114); alignment <= 256 is always met. */
int32_t kxc_hip_alloc(int32_t device_id, size_t nbytes, size_t alignment, void** out_ptr);
int32_t kxc_hip_free(int32_t device_id, void* ptr);
/* CopyDataFromTo with offsets and stream (cuda_device_api.cc:122-157).
 * kind: 0 host->device, 1 device->host, 2 device->device, 3 host->host.
 * stream NULL and no current stream: synchronous copy. */
int32_t kxc_hip_copy(const void* from, size_t from_offset, void* to, size_t to_offset,
                     size_t nbytes, int32_t kind, int32_t device_id, void* stream);
/* CreateStream / FreeStream / SetStream / GetCurrentStream / StreamSync /
 * SyncStreamFromTo (cuda_device_api.cc:223-328).  The current stream is per thread.
 * kxc_hip_stream_sync(dev, NULL) with no current stream synchronises the whole device. */
int32_t kxc_hip_stream_create(int32_t device_id, void** out_stream);
int32_t kxc_hip_stream_destroy(int32_t device_id, void* stream);
int32_t kxc_hip_set_stream(int32_t device_id, void* stream);
int32_t kxc_hip_get_stream(int32_t device_id, void** out_stream);
int32_t kxc_hip_stream_sync(int32_t device_id, void* stream);
int32_t kxc_hip_stream_wait(int32_t device_id, void* src_stream, void* dst_stream);

/* Fill (the reference's only GPU test uses cudaMemsetAsync beside the device API, test/cupti_smoke_test.cpp:113-118):
 * every byte of [ptr, ptr + nbytes) = value & 0xff; stream NULL and no current stream: synchronous.  On a stream
 * that is being captured into a graph the fill is a small kernel, not a memset node. */
int32_t kxc_hip_memset(void* ptr, int32_t value, size_t nbytes, int32_t device_id, void* stream);
/* Number of device allocations (hipMalloc: data spaces, plan workspaces, split-reduction scratch) this library has
 * made in the process so far.  No counterpart in the reference; lets a caller that must not allocate -- and the test
 * of the entry point that allocates nothing -- check that a call did not. */
int64_t kxc_hip_debug_device_allocations(void);

/* Activity records for the profiling bundle: what the reference's CUPTI adapter collects for CUDA
 * (src/base/profiling.cc:537-651: runtime API calls, memcpy, memset, kernels, each with start and end), taken at
 * the library's own call sites.  While enabled, every HIP runtime call made by section 1 (device API) and section 3
 * (module loader) leaves a RUNTIME_API record timed on the host, and every copy, fill and kernel launch they enqueue
 * leaves a MEMCPY / MEMSET / KERNEL record timed on the GPU by two HIP events on its stream (timed_on_gpu = 1;
 * synchronous copies are timed on the host).  Times are nanoseconds of the clock kxc_hip_activity_now_ns() reads.
 * correlation_id ties a device record to the API record of the call that enqueued it.  kxc_hip_activity_drain
 * hands over and forgets the finished records, waiting for device records still in flight; capacity 0 only counts.
 * At most 65536 device records wait for a drain; later ones are dropped until it comes.
 *
 * kxc_hip_activity_enable(mode): 0 off; 1 the call sites of this library, as above; 2 the records come from
 * rocprofiler-sdk's buffered tracing instead (kernel dispatches, memory copies, HIP runtime calls of the WHOLE
 * process -- also those the application or another library makes -- timed by the profiler: timed_on_gpu = 2; fills
 * appear as the runtime call and the fill kernel, there is no MEMSET record).  Mode 2 loads
 * libkxc_hip_rocprof.so from this library's directory, a rocprofiler-sdk tool (it exports rocprofiler_configure),
 * and registers it with rocprofiler_force_configure; that only works BEFORE the process's first HIP call, so either
 * call kxc_hip_activity_enable(2) first thing, or set KXC_PROFILE_GPU_ACTIVITY=2 in the environment (the tool is
 * then registered while this library loads), or list the tool library in ROCP_TOOL_LIBRARIES.  Too late is an
 * error that says so; mode 1 still works then. */
#define KXC_HIP_ACTIVITY_RUNTIME_API 0
#define KXC_HIP_ACTIVITY_MEMCPY 1
#define KXC_HIP_ACTIVITY_MEMSET 2
#define KXC_HIP_ACTIVITY_KERNEL 3
typedef struct kxc_hip_activity_record {
    int32_t kind;                    /* KXC_HIP_ACTIVITY_* */
    char name[96];                   /* HIP runtime call, or kernel symbol */
    int64_t start_ns, end_ns;
    int64_t bytes;                   /* copies and fills */
    int32_t value;                   /* fills */
    int32_t copy_kind;               /* copies: 0 host->device, 1 device->host, 2 device->device, 3 host->host */
    uint32_t grid[3], block[3];      /* kernels */
    uint32_t dynamic_shared_memory;
    uint64_t correlation_id;
    int32_t return_value;            /* RUNTIME_API: hipError_t of the call */
    int32_t device_id;
    uint64_t stream;
    uint64_t thread_id;
    int32_t timed_on_gpu;
} kxc_hip_activity_record;
int32_t kxc_hip_activity_enable(int32_t enable);
int32_t kxc_hip_activity_drain(kxc_hip_activity_record* records, int32_t capacity, int32_t* count);
int64_t kxc_hip_activity_now_ns(void);

/* ========================================================================
 * 2. Hand-written operators.  Each is the GPU implementation of one
 *    FRelayToTE compute definition (the CPU definition stays the fallback).
 * ===================================================================== */

#define KXC_HIP_CONV_BIAS 1u       /* + bias[o]              (convolution.cc:72-74)            */
#define KXC_HIP_CONV_RESIDUAL 2u   /* + residual[n,o,h,w]    (add(conv_out, skip), math.cc:41-47) */
#define KXC_HIP_CONV_RELU 4u       /* (v > 0) ? v : 0        (nn.h:19-30)                      */
#define KXC_HIP_CONV_HPOOL 0x10u   /* y is max-pooled along W on the way out; see kxc_hip_conv2d_hpool_supported */
#define KXC_HIP_CONV_FORCE_DIRECT 0x100u /* use the one-thread-per-output kernel (reference order) */

/* nn_conv2d: Conv2DCompute (src/relay/op/nn/convolution.cc:38-75) ->
 * topi::conv2d_nchw (include/te/topi/nn.h:107-158); shapes by Conv2DInferType
 * (src/relay/type_infer.cc:346-400).  x [n,c,h,w], w [o,c,kh,kw], y [n,o,oh,ow].
 * The fused epilogue applies, in the reference chain's order, bias, residual
 * add (conv_out + residual), ReLU; each one rounded fp32 operation. */
typedef struct kxc_hip_conv2d_desc {
    int32_t n, c, h, w;
    int32_t o, kh, kw;
    int32_t stride_h, stride_w;
    int32_t pad_h, pad_w;            /* padding[0], padding[1], applied to both sides (convolution.cc:53-54) */
    int32_t dil_h, dil_w;
    uint32_t flags;
} kxc_hip_conv2d_desc;
int32_t kxc_hip_conv2d_nchw_f32(const kxc_hip_conv2d_desc* desc, const float* x, const float* w,
                                const float* bias, const float* residual, float* y, void* stream);
/* Name of the kernel variant the library would launch for this shape ("mfma_..." or "direct"). */
const char* kxc_hip_conv2d_variant(const kxc_hip_conv2d_desc* desc);
/* The same operator for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, kernels and results
 * as kxc_hip_conv2d_nchw_f32, but it calls no hipMalloc / hipFree or allocating library routine: the partial sums
 * of a reduction split over workgroups (small launches with long reductions, e.g. batch-1 512-channel layers) go
 * to a device array built into the library, kxc_hip_conv2d_noalloc_scratch_bytes() = 8 MiB per GPU, held until the
 * process ends.  A launch whose partial sums would not fit fails with KXC_HIP_ERR_INVALID and launches nothing
 * (the library's own choice of split never exceeds the array; only a forced split can).  All calls on one GPU
 * share that array: two calls whose kernels may overlap on that GPU (different streams, different threads) race;
 * calls enqueued on one stream are safe. */
int32_t kxc_hip_conv2d_nchw_f32_noalloc(const kxc_hip_conv2d_desc* desc, const float* x, const float* w,
                                        const float* bias, const float* residual, float* y, void* stream);
size_t kxc_hip_conv2d_noalloc_scratch_bytes(void);
/* Bytes of scratch (partial sums) a launch for this shape uses, 0 when its reduction is not split over workgroups:
 * lets a caller see beforehand whether kxc_hip_conv2d_nchw_f32_noalloc takes the shape. */
int32_t kxc_hip_conv2d_scratch_needed(const kxc_hip_conv2d_desc* desc, size_t* out_bytes);

/* Two nn_conv2d calls on the same input in one launch: the convolution `desc` describes (convolution.cc:38-75, with
 * its fused epilogue as above) and a 1x1 convolution with the same strides, no padding and the same number of
 * output channels, y2[n,o,oh,ow] = sum_c x[n,c,oh*stride_h,ow*stride_w] * w2[o,c] (+ bias2[o], NULL = none) -- a
 * residual block's first 3x3/2 convolution and its 1x1/2 downsample (test/resnet18_ir_dump.cpp:330-352).  The 1x1
 * operand is the tap (pad/dilation) of the first convolution's window, which its staged input already holds, so
 * the input is read once and the second launch disappears.  Both outputs equal what the two separate calls give
 * (the second one bit for bit: same kernel arithmetic) unless the launch is small enough to split its reduction
 * over workgroups: then the parts of both outputs are added in split order by one adding launch, within the fp32
 * tolerance of the separate calls (KXC_HIP_PAIR_SPLIT=0: such shapes are reported unsupported instead).
 *   ..._supported: 1 when a matrix-core kernel with a second output covers the shape (padding a multiple of the
 *   dilation and inside the filter, and "same" padding -- 2*pad = dilation*(k-1) -- so that the unpadded 1x1
 *   convolution has the first one's output extent; no 1x1 first filter), else 0; ..._variant names it ("unsupported" otherwise). */
int32_t kxc_hip_conv2d_pair_supported(const kxc_hip_conv2d_desc* desc);
const char* kxc_hip_conv2d_pair_variant(const kxc_hip_conv2d_desc* desc);
int32_t kxc_hip_conv2d_pair_nchw_f32(const kxc_hip_conv2d_desc* desc, const float* x, const float* w,
                                     const float* bias, const float* residual, float* y, const float* w2,
                                     const float* bias2, float* y2, void* stream);

/* nn_conv2d -> nn_relu -> nn_max_pool2d(3x3, stride 2, padding 1) (test/resnet18_ir_dump.cpp:281-291; MaxPool2DCompute,
 * src/relay/op/nn/pooling.cc:50-67 -> topi::pool2d, include/te/topi/nn.h:161-258): a maximum over a 3x3 window is
 * the maximum over three rows of the maxima over three columns, so the convolution kernel can take the column
 * maxima while an output row is still in registers.  With KXC_HIP_CONV_HPOOL in desc->flags
 * (kxc_hip_conv2d_nchw_f32 and kxc_hip_plan_add_conv2d) y is [n,o,oh,ow/2] with
 *   y[n,o,oh,pw] = max(v[2pw-1], v[2pw], v[2pw+1]),  v = relu(conv + bias) of row (n,o,oh),  v[-1] left out,
 * half the bytes of the unpooled map; kxc_hip_pool2d_f32 with a 3x1 window, stride (2,1) and padding (1,0,1,0)
 * finishes the pool.  Every value is a ReLU result (>= +0, never NaN), so the pooling pad candidate of the
 * reference never wins and the two-step maximum equals the 3x3 one bit for bit.
 *   ..._supported: 1 when a kernel with that epilogue covers the shape: KXC_HIP_CONV_RELU set, no residual, output
 *   channels a multiple of 8, an even output width that divides the kernel's 224-pixel tile (7x7 filters: 112, 56, 32, 16 ...), n*oh*ow a multiple of 224.
 *   ..._preferred: ... and the library expects conv + column pool to beat conv + 3x3 pool (KXC_HIP_CONV_HPOOL=0/1 in
 *   the environment overrides the rule). */
int32_t kxc_hip_conv2d_hpool_supported(const kxc_hip_conv2d_desc* desc);
int32_t kxc_hip_conv2d_hpool_preferred(const kxc_hip_conv2d_desc* desc);

/* nn_conv2d with a 3x3 filter, stride 1, dilation 1 and c % 4 == 0 as Winograd F(2x2, 3x3) on the matrix cores:
 * same operator and epilogue as kxc_hip_conv2d_nchw_f32 (convolution.cc:38-75, nn.h:107-158) with 2.25x fewer
 * multiplies; the sums are formed in a different order, results agree within the operator's fp32 tolerance.
 * The filter is passed in transformed form: `u` holds weight_bytes bytes written by ..._transform_weights from
 * the OIHW tensor (the reference keeps weights as module constants, CompiledModule::GetConstants,
 * include/compiler.h:83, so a caller transforms them once per module).
 *   ..._supported: 1 when the shape qualifies, else 0 (no error is recorded). */
int32_t kxc_hip_conv2d_winograd_supported(const kxc_hip_conv2d_desc* desc);
int32_t kxc_hip_conv2d_winograd_weight_bytes(const kxc_hip_conv2d_desc* desc, size_t* out_bytes);
int32_t kxc_hip_conv2d_winograd_transform_weights(const kxc_hip_conv2d_desc* desc, const float* w_oihw, float* u,
                                                  void* stream);
int32_t kxc_hip_conv2d_winograd_nchw_f32(const kxc_hip_conv2d_desc* desc, const float* x, const float* u,
                                         const float* bias, const float* residual, float* y, void* stream);
const char* kxc_hip_conv2d_winograd_variant(const kxc_hip_conv2d_desc* desc);
/* 1 when the shape qualifies and this path is expected to beat kxc_hip_conv2d_nchw_f32, else 0.  Measured on
 * MI355X it does for every ResNet-18 layer from batch 1 to 64 (small launches split their input channels over
 * workgroups and finish in a second, adding kernel), so by default every supported shape is preferred; the
 * environment variable KXC_HIP_WINOGRAD_MIN_WORK = f restricts it to 2x2 output blocks * o >= f * c. */
int32_t kxc_hip_conv2d_winograd_preferred(const kxc_hip_conv2d_desc* desc);

/* nn_relu: ReluCompute (src/relay/op/nn/activation.cc:14-19). */
int32_t kxc_hip_relu_f32(const float* x, float* y, int64_t n, void* stream);
/* add / subtract / multiply / divide: broadcast.h:90-113 via math.cc:41-95.
 * op 0..3; shapes right-aligned, ndim <= 6; relu != 0 fuses a following nn_relu. */
int32_t kxc_hip_broadcast_binary_f32(int32_t op, const float* a, const int64_t* a_shape, int32_t a_ndim,
                                     const float* b, const int64_t* b_shape, int32_t b_ndim,
                                     float* y, int32_t relu, void* stream);
/* T_conv2d_bias_add on its own (convolution.cc:72-74): y[n,o,:] = x[n,o,:] + bias[o]. */
int32_t kxc_hip_bias_add_nchw_f32(const float* x, const float* bias, float* y,
                                  int64_t n, int64_t o, int64_t hw, int32_t relu, void* stream);

/* nn_max_pool2d / nn_avg_pool2d: MaxPool2DCompute / AvgPool2DCompute
 * (src/relay/op/nn/pooling.cc:50-86) -> topi::pool2d (nn.h:161-258). */
typedef struct kxc_hip_pool2d_desc {
    int32_t n, c, h, w;
    int32_t kh, kw, stride_h, stride_w;
    int32_t pad_top, pad_left, pad_bottom, pad_right;
    int32_t ceil_mode;
    int32_t is_avg;                  /* 0 max, 1 avg */
} kxc_hip_pool2d_desc;
int32_t kxc_hip_pool2d_f32(const kxc_hip_pool2d_desc* desc, const float* x, float* y, void* stream);

/* nn_global_avg_pool2d: GlobalAvgPool2DCompute (pooling.cc:88-98) -> nn.h:260-287. */
int32_t kxc_hip_global_avg_pool2d_f32(const float* x, float* y, int64_t n, int64_t c, int64_t h,
                                      int64_t w, void* stream);

/* nn_dense (DenseCompute, src/relay/op/nn/dense.cc:27-32) and nn_gemm (GemmCompute :34-61):
 * y[m,n] = alpha * sum_k a[m,k]*b[n,k] (transB=1) or a[m,k]*b[k,n] (transB=0), + beta*c[n].
 * c may be NULL (nn_dense); c_len is n or 1. */
int32_t kxc_hip_gemm_f32(const float* a, const float* b, const float* c, float* y,
                         int64_t m, int64_t n, int64_t k, float alpha, float beta,
                         int32_t transB, int64_t c_len, void* stream);

/* nn_flatten (FlattenCompute, src/relay/op/tensor/transform.cc:140-182): a row-major copy.
 * (Inside a launch plan a flatten is an alias and launches nothing.) */
int32_t kxc_hip_flatten_f32(const float* x, float* y, int64_t n, void* stream);

/* ---- int8 family.  The reference has no quantised operator; these implement the
 *      definition in oracle/kxc_oracle.h (qnn-style conv/dense with int32 accumulate and
 *      per-output-channel fp32 requantisation, round half to even). ---- */
int32_t kxc_hip_quantize_f32_i8(const float* x, int8_t* q, int64_t n, float scale, void* stream);
/* Calibration helper: *out (device float) = max |x[i]| (0 for an empty tensor; NaN ignored).  Per-tensor
 * symmetric scales are max-abs / 127. */
int32_t kxc_hip_absmax_f32(const float* x, int64_t n, float* out, void* stream);
typedef struct kxc_hip_qconv2d_desc {
    int32_t n, c, h, w;
    int32_t o, kh, kw;
    int32_t stride_h, stride_w;
    int32_t pad_h, pad_w;
    uint32_t flags;                  /* KXC_HIP_CONV_BIAS | _RESIDUAL | _RELU | _HPOOL | _FORCE_DIRECT */
    float res_mult;
} kxc_hip_qconv2d_desc;
int32_t kxc_hip_qconv2d_nchw_i8(const kxc_hip_qconv2d_desc* desc, const int8_t* x, const int8_t* w,
                                const int32_t* bias, const float* mult, const int8_t* residual,
                                int8_t* y, void* stream);
int32_t kxc_hip_qdense_i8(const int8_t* a, const int8_t* b, const int32_t* bias, const float* mult,
                          float* y, int64_t m, int64_t n, int64_t k, void* stream);
int32_t kxc_hip_maxpool2d_i8(const kxc_hip_pool2d_desc* desc, const int8_t* x, int8_t* y, void* stream);
int32_t kxc_hip_global_avg_pool2d_i8(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t h,
                                     int64_t w, float mult, void* stream);

/* ---- int8 on the channel-blocked "c16" layout: logical [N,C,H,W] stored as [N][ceil(C/16)][H][W][16]
 *      (element (n,c,h,w) at (((n*CB + c/16)*H + h)*W + w)*16 + c%16, channels >= C are zero).  One pixel's 16
 *      channels are the 16-byte k-slice a lane feeds to v_mfma_i32_32x32x32_i8, so the convolution runs on
 *      the int8 matrix cores with no byte gathers.  Same arithmetic as the NCHW entry points; like them these
 *      have no counterpart in the reference (no int8 operator exists there). ---- */
/* Size in bytes of the packed weight buffer for a convolution (output channels must be a multiple of 32). */
int32_t kxc_hip_qconv2d_c16_packed_bytes(const kxc_hip_qconv2d_desc* desc, size_t* out_bytes);
/* Repack OIHW int8 weights (device) into the order the matrix-core kernel reads them (device, once per model). */
int32_t kxc_hip_qconv2d_c16_pack_weights(const kxc_hip_qconv2d_desc* desc, const int8_t* w_oihw, int8_t* packed,
                                         void* stream);
/* Name of the kernel variant the shape selects ("none" when no matrix-core variant covers it). */
const char* kxc_hip_qconv2d_c16_variant(const kxc_hip_qconv2d_desc* desc);
/* 1 when a matrix-core variant covers the shape (what an operator hook asks before it chooses the layout). */
int32_t kxc_hip_qconv2d_c16_supported(const kxc_hip_qconv2d_desc* desc);
/* x, residual, y in c16; w_packed from kxc_hip_qconv2d_c16_pack_weights; bias int32[O], mult float[O]. */
int32_t kxc_hip_qconv2d_c16_i8(const kxc_hip_qconv2d_desc* desc, const int8_t* x, const int8_t* w_packed,
                               const int32_t* bias, const float* mult, const int8_t* residual, int8_t* y,
                               void* stream);
/* Two outputs from one launch (a residual block's first 3x3/2 convolution and its 1x1/2 downsample): y as above, and
 * y2[n,o,oh,ow] = requantise(sum_c x[n,c,oh*stride,ow*stride] * w2[o,c] + bias2[o], mult2[o]) without ReLU -- the 1x1
 * convolution with the same strides and no padding, whose operand is the tap (pad_h, pad_w) of the first one's window
 * (needs "same" padding, 2*pad = k-1, so that both convolutions have the same output extent).  w2_packed comes from kxc_hip_qconv2d_c16_pair_pack_weights (w2 is [o,c,1,1], packed in
 * the chunking of `desc`); bias2 may be NULL.  Bit-identical to the two separate launches. */
int32_t kxc_hip_qconv2d_c16_pair_supported(const kxc_hip_qconv2d_desc* desc);
int32_t kxc_hip_qconv2d_c16_pair_packed_bytes(const kxc_hip_qconv2d_desc* desc, size_t* out_bytes);
int32_t kxc_hip_qconv2d_c16_pair_pack_weights(const kxc_hip_qconv2d_desc* desc, const int8_t* w2_oihw, int8_t* packed,
                                              void* stream);
int32_t kxc_hip_qconv2d_c16_pair_i8(const kxc_hip_qconv2d_desc* desc, const int8_t* x, const int8_t* w_packed,
                                    const int32_t* bias, const float* mult, const int8_t* residual, int8_t* y,
                                    const int8_t* w2_packed, const int32_t* bias2, const float* mult2, int8_t* y2,
                                    void* stream);
/* Layout converters and the quantising converter (fp32 NCHW -> int8 c16, same rounding as kxc_hip_quantize_f32_i8). */
int32_t kxc_hip_i8_nchw_to_c16(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t hw, void* stream);
int32_t kxc_hip_i8_c16_to_nchw(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t hw, void* stream);
int32_t kxc_hip_quantize_f32_nchw_to_c16_i8(const float* x, int8_t* y, int64_t n, int64_t c, int64_t hw,
                                            float scale, void* stream);
/* First layer (7x7, stride 2, padding 3, at most 4 input channels, width a multiple of 4) on the "c4" input
 * layout [N][H][W][4] (4 bytes per pixel, channels >= C zero): a k-step of the matrix instruction is one
 * filter row of 8 taps x 4 channels.  Output is c16.  Weights are packed by the _c4_pack_weights call. */
int32_t kxc_hip_qconv2d_c4_supported(const kxc_hip_qconv2d_desc* desc);
int32_t kxc_hip_qconv2d_c4_packed_bytes(const kxc_hip_qconv2d_desc* desc, size_t* out_bytes);
int32_t kxc_hip_qconv2d_c4_pack_weights(const kxc_hip_qconv2d_desc* desc, const int8_t* w_oihw, int8_t* packed,
                                        void* stream);
int32_t kxc_hip_qconv2d_c4_i8(const kxc_hip_qconv2d_desc* desc, const int8_t* x_c4, const int8_t* w_packed,
                              const int32_t* bias, const float* mult, int8_t* y_c16, void* stream);
/* The same first layer followed by nn_max_pool2d with a 3x3 window, stride 2 and padding 1 on all sides (the
 * chain of test/resnet18_ir_dump.cpp:281-291 in its int8 form) as ONE kernel: y_c16 is the pooled map
 * [n, o, (oh-1)/2+1, (ow-1)/2+1] in c16, bit for bit what kxc_hip_qconv2d_c4_i8 followed by kxc_hip_maxpool2d_c16_i8
 * gives (the padding candidate of the int8 pool is -128); the unpooled map is never written.  ..._supported: the
 * first-layer conditions and a pooled width of at most 60 columns. */
int32_t kxc_hip_qconv2d_c4_maxpool_supported(const kxc_hip_qconv2d_desc* desc);
int32_t kxc_hip_qconv2d_c4_maxpool_i8(const kxc_hip_qconv2d_desc* desc, const int8_t* x_c4, const int8_t* w_packed,
                                      const int32_t* bias, const float* mult, int8_t* y_c16, void* stream);
int32_t kxc_hip_quantize_f32_nchw_to_c4_i8(const float* x, int8_t* y, int64_t n, int64_t c, int64_t hw,
                                           float scale, void* stream);
int32_t kxc_hip_maxpool2d_c16_i8(const kxc_hip_pool2d_desc* desc, const int8_t* x, int8_t* y, void* stream);
/* Output is [N][ceil(C/16)*16] int8 (c16 with H = W = 1, i.e. plain row-major when C is a multiple of 16). */
int32_t kxc_hip_global_avg_pool2d_c16_i8(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t h,
                                         int64_t w, float mult, void* stream);

/* ========================================================================
 * 3. Module loader -- run-time compiled kernels (the TIR->HIP emitter's output).
 *    Mirrors the only device-code launch site in the reference, an NVRTC +
 *    cuLaunchKernel sequence (test/cupti_smoke_test.cpp:143-205), and is what a
 *    HIP CompiledKernelNode (include/codegen/compiled_kernel.h:19-41) owns.
 * ===================================================================== */
typedef struct kxc_hip_module kxc_hip_module;   /* opaque */
/* hipRTC-compile `source` for gfx950 and load it.  log (may be NULL) receives the compiler log. */
int32_t kxc_hip_module_compile(const char* source, const char* name, kxc_hip_module** out,
                               char* log, size_t log_capacity);
/* Compile only (no GPU needed): code object size in *out_size; used by build-time checks. */
int32_t kxc_hip_module_compile_only(const char* source, const char* name, size_t* out_size,
                                    char* log, size_t log_capacity);
int32_t kxc_hip_module_get_function(kxc_hip_module* module, const char* symbol, void** out_function);
/* hipModuleLaunchKernel(f, grid, block, shared_bytes, stream, kernel_params, NULL). */
int32_t kxc_hip_module_launch(void* function, const uint32_t grid[3], const uint32_t block[3],
                              uint32_t shared_bytes, void* stream, void** kernel_params);
int32_t kxc_hip_module_free(kxc_hip_module* module);

/* ========================================================================
 * 4. Launch plan -- the kernel-launch half of the reference's ExecutionPlan
 *    (include/base/execution_plan.h:42-50,102-130; its executor only copies
 *    buffers, src/base/disco/executor.cc:122-157).  One plan = the body of one
 *    compiled function `int32_t kxc_kernel_main(void** packed_args)`
 *    (src/codegen/compiled_kernel.cc:41-55): a list of launches on ONE stream
 *    over buffers that are either caller arguments or slots of a workspace the
 *    plan owns (allocated once, no per-run allocation).
 * ===================================================================== */
typedef struct kxc_hip_plan kxc_hip_plan;       /* opaque */

/* A buffer operand: packed_args[index] (kind 0), byte offset into the plan
 * workspace (kind 1), absent (kind 2, e.g. no bias), or packed_args[index] plus a byte offset that is a
 * multiple of 16 (kind 3, index_or_offset = KXC_HIP_ARG_OFFSET(index, bytes): one share of a batched
 * argument). */
typedef struct kxc_hip_buf {
    int32_t kind;
    int64_t index_or_offset;
} kxc_hip_buf;
#define KXC_HIP_BUF_ARG 0
#define KXC_HIP_BUF_WORKSPACE 1
#define KXC_HIP_BUF_NONE 2
#define KXC_HIP_BUF_ARG_OFFSET 3
#define KXC_HIP_ARG_OFFSET(index, bytes) (((int64_t)(index) << 48) | (int64_t)(bytes))   /* index < 32768, bytes < 2^48 */

int32_t kxc_hip_plan_create(int32_t device_id, int32_t num_packed_args, kxc_hip_plan** out);
int32_t kxc_hip_plan_destroy(kxc_hip_plan* plan);
/* Node builders; `symbol` is stored as KernelExecNode::kernel_symbol would be. */
int32_t kxc_hip_plan_add_conv2d(kxc_hip_plan* plan, const kxc_hip_conv2d_desc* desc, kxc_hip_buf x,
                                kxc_hip_buf w, kxc_hip_buf bias, kxc_hip_buf residual, kxc_hip_buf y);
/* The same operator through kxc_hip_conv2d_winograd_nchw_f32.  `w` is the OIHW weight tensor as the reference
 * passes it (a module constant among the packed arguments); `u` is a workspace region of
 * kxc_hip_conv2d_winograd_weight_bytes bytes that no other node uses.
 * By default every run starts with ONE launch that transforms the weights of all the plan's Winograd nodes from
 * the pointers passed to that run, so a run always sees the current contents of its constants, like the CPU
 * backend, which re-reads every constant on every call (src/codegen/compiled_kernel.cc:41-55).
 * kxc_hip_plan_freeze_constants(plan, 1) is the serving mode: the caller promises that the weight tensors do not
 * change; they are transformed when first seen and again only when a different pointer arrives (a run on another
 * stream is ordered after the transforms), and kxc_hip_plan_invalidate_constants forces a new transform after an
 * in-place update. */
int32_t kxc_hip_plan_add_conv2d_winograd(kxc_hip_plan* plan, const kxc_hip_conv2d_desc* desc, kxc_hip_buf x,
                                         kxc_hip_buf w, kxc_hip_buf bias, kxc_hip_buf residual, kxc_hip_buf y,
                                         kxc_hip_buf u);
/* Both convolutions of kxc_hip_conv2d_pair_nchw_f32 as one node. */
int32_t kxc_hip_plan_add_conv2d_pair(kxc_hip_plan* plan, const kxc_hip_conv2d_desc* desc, kxc_hip_buf x,
                                     kxc_hip_buf w, kxc_hip_buf bias, kxc_hip_buf residual, kxc_hip_buf y,
                                     kxc_hip_buf w2, kxc_hip_buf bias2, kxc_hip_buf y2);
int32_t kxc_hip_plan_invalidate_constants(kxc_hip_plan* plan);
int32_t kxc_hip_plan_freeze_constants(kxc_hip_plan* plan, int32_t frozen);
int32_t kxc_hip_plan_add_pool2d(kxc_hip_plan* plan, const kxc_hip_pool2d_desc* desc, kxc_hip_buf x,
                                kxc_hip_buf y);
int32_t kxc_hip_plan_add_global_avg_pool2d(kxc_hip_plan* plan, int64_t n, int64_t c, int64_t h,
                                           int64_t w, kxc_hip_buf x, kxc_hip_buf y);
int32_t kxc_hip_plan_add_gemm(kxc_hip_plan* plan, int64_t m, int64_t n, int64_t k, float alpha,
                              float beta, int32_t transB, int64_t c_len, kxc_hip_buf a,
                              kxc_hip_buf b, kxc_hip_buf c, kxc_hip_buf y);
int32_t kxc_hip_plan_add_binary(kxc_hip_plan* plan, int32_t op, const int64_t* a_shape,
                                int32_t a_ndim, const int64_t* b_shape, int32_t b_ndim, int32_t relu,
                                kxc_hip_buf a, kxc_hip_buf b, kxc_hip_buf y);
int32_t kxc_hip_plan_add_relu(kxc_hip_plan* plan, int64_t n, kxc_hip_buf x, kxc_hip_buf y);
int32_t kxc_hip_plan_add_copy(kxc_hip_plan* plan, int64_t nbytes, kxc_hip_buf x, kxc_hip_buf y);
int32_t kxc_hip_plan_add_qconv2d(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x,
                                 kxc_hip_buf w, kxc_hip_buf bias, kxc_hip_buf mult,
                                 kxc_hip_buf residual, kxc_hip_buf y);
int32_t kxc_hip_plan_add_quantize(kxc_hip_plan* plan, int64_t n, float scale, kxc_hip_buf x, kxc_hip_buf q);
int32_t kxc_hip_plan_add_maxpool2d_i8(kxc_hip_plan* plan, const kxc_hip_pool2d_desc* desc,
                                      kxc_hip_buf x, kxc_hip_buf y);
int32_t kxc_hip_plan_add_global_avg_pool2d_i8(kxc_hip_plan* plan, int64_t n, int64_t c, int64_t h,
                                              int64_t w, float mult, kxc_hip_buf x, kxc_hip_buf y);
int32_t kxc_hip_plan_add_qconv2d_c16(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x,
                                     kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult,
                                     kxc_hip_buf residual, kxc_hip_buf y);
/* The c16 convolution with the second output of kxc_hip_qconv2d_c16_pair_i8 as one node. */
int32_t kxc_hip_plan_add_qconv2d_c16_pair(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x,
                                          kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult,
                                          kxc_hip_buf residual, kxc_hip_buf y, kxc_hip_buf w2_packed,
                                          kxc_hip_buf bias2, kxc_hip_buf mult2, kxc_hip_buf y2);
int32_t kxc_hip_plan_add_qconv2d_c4(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x_c4,
                                    kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf y_c16);
/* kxc_hip_qconv2d_c4_maxpool_i8 as a plan node: y_c16 is the pooled map. */
int32_t kxc_hip_plan_add_qconv2d_c4_maxpool(kxc_hip_plan* plan, const kxc_hip_qconv2d_desc* desc, kxc_hip_buf x_c4,
                                            kxc_hip_buf w_packed, kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf y_c16);
int32_t kxc_hip_plan_add_quantize_c4(kxc_hip_plan* plan, int64_t n, int64_t c, int64_t hw, float scale,
                                     kxc_hip_buf x, kxc_hip_buf q);
int32_t kxc_hip_plan_add_quantize_c16(kxc_hip_plan* plan, int64_t n, int64_t c, int64_t hw, float scale,
                                      kxc_hip_buf x, kxc_hip_buf q);
int32_t kxc_hip_plan_add_maxpool2d_c16_i8(kxc_hip_plan* plan, const kxc_hip_pool2d_desc* desc,
                                          kxc_hip_buf x, kxc_hip_buf y);
int32_t kxc_hip_plan_add_global_avg_pool2d_c16_i8(kxc_hip_plan* plan, int64_t n, int64_t c, int64_t h,
                                                  int64_t w, float mult, kxc_hip_buf x, kxc_hip_buf y);
int32_t kxc_hip_plan_add_qdense(kxc_hip_plan* plan, int64_t m, int64_t n, int64_t k, kxc_hip_buf a,
                                kxc_hip_buf b, kxc_hip_buf bias, kxc_hip_buf mult, kxc_hip_buf y);
/* kxc_hip_i8_nchw_to_c16 (to_c16 != 0) or kxc_hip_i8_c16_to_nchw as a node: what a graph compiler places on an edge
 * between an operator that keeps int8 activations in NCHW and one that keeps them channel-blocked. */
int32_t kxc_hip_plan_add_i8_layout(kxc_hip_plan* plan, int32_t to_c16, int64_t n, int64_t c, int64_t hw,
                                   kxc_hip_buf x, kxc_hip_buf y);
/* Constant preparation: the OIHW int8 weights `w_oihw` of a convolution (a packed argument: a module constant,
 * include/relay/relay.h:120-134, which the caller passes again on every run, test/onnx_importer_test.cpp:249-255)
 * are packed into the workspace region `w_packed` in the order kind's kernel reads them --
 * KXC_HIP_QPACK_C16: kxc_hip_qconv2d_c16_pack_weights, _C4: kxc_hip_qconv2d_c4_pack_weights, _C16_PAIR:
 * kxc_hip_qconv2d_c16_pair_pack_weights (desc = the first convolution, w_oihw = the second one's [o,c,1,1]).
 * Like the Winograd filter transforms, all packs of a plan run as ONE launch at the start of every run, so a run
 * sees the current contents of its constants; with kxc_hip_plan_freeze_constants a tensor is packed when its
 * pointer is first seen (every_run != 0 keeps a pack on every run even then: weights that are not constants). */
#define KXC_HIP_QPACK_C16 1
#define KXC_HIP_QPACK_C4 2
#define KXC_HIP_QPACK_C16_PAIR 3
int32_t kxc_hip_plan_add_qconv_weight_pack(kxc_hip_plan* plan, int32_t kind, const kxc_hip_qconv2d_desc* desc,
                                           kxc_hip_buf w_oihw, kxc_hip_buf w_packed, int32_t every_run);
int32_t kxc_hip_plan_num_weight_packs(const kxc_hip_plan* plan);
/* A run-time compiled kernel (section 3): params[i] is a buffer operand, passed as a pointer. */
int32_t kxc_hip_plan_add_module_kernel(kxc_hip_plan* plan, void* function, const char* symbol,
                                       const uint32_t grid[3], const uint32_t block[3],
                                       uint32_t shared_bytes, const kxc_hip_buf* params,
                                       int32_t num_params);
/* Text form of a finalized plan (every launch with its descriptor, operands and geometry), so that a compiled
 * function can be stored and run again without compiling: the launch-level counterpart of the reference's
 * execution-plan JSON (src/base/execution_plan.cc:674-877), which keeps only value ids and kernel_symbol.
 * With buffer == NULL only *needed is set.  Deserialising allocates the workspace on device_id; generated
 * kernels are looked up by name in `modules` (compiled by the caller from the saved source). */
int32_t kxc_hip_plan_serialize(const kxc_hip_plan* plan, char* buffer, size_t capacity, size_t* needed);
int32_t kxc_hip_plan_deserialize(const char* text, int32_t device_id, kxc_hip_module* const* modules,
                                 int32_t num_modules, kxc_hip_plan** out_plan);
/* Concurrency inside a plan.  lane = 1 puts node `node` (index in order of the add calls) on the plan's side
 * stream: it starts after everything added before it and runs concurrently with the main-lane nodes added
 * after it.  join = 1 on a main-lane node makes it wait first for every side-lane node added before it.  The
 * caller guarantees that no main-lane node between a side node and its join reads the side node's output or
 * overwrites a buffer the side node uses.  Without a join the plan run ends with one.  (Independent branches of
 * a graph -- a residual block's 1x1 downsample next to its 3x3 convolution -- overlap this way.) */
int32_t kxc_hip_plan_set_concurrency(kxc_hip_plan* plan, int32_t node, int32_t lane, int32_t join);
/* Chains: independent runs of nodes inside one plan, e.g. the same network on the two halves of a batch (their
 * operands are workspace regions of their own and KXC_HIP_BUF_ARG_OFFSET shares of the arguments).  Nodes with
 * chain k in [1, 7] run on the plan's k-th chain stream in the order they were added, from the start of a plan
 * run (after everything enqueued before it on the caller's stream) to its end (the caller's stream then waits for
 * every chain); nodes with chain 0 run on the caller's stream as before.  Under graph replay the chains are
 * parallel branches of the captured graph.  A launch on a machine that other launches fill needs no split
 * reduction or small tile of its own to fill it: kxc_hip_plan_set_select_lanes(plan, n) makes finalize choose
 * every convolution variant as for n equal launches side by side, and kxc_hip_set_select_lanes(n) does the same
 * for the calling thread's variant queries (kxc_hip_conv2d_variant, _pair_supported, _winograd_preferred ...)
 * and stand-alone launches; it returns the previous value.  No counterpart in the reference, whose executor runs
 * one node after the other (src/base/disco/executor.cc:59-90). */
int32_t kxc_hip_plan_set_chain(kxc_hip_plan* plan, int32_t node, int32_t chain);
/* Reorders the nodes so that a run enqueues the k-th node of the main lane, then the k-th node of every chain, then
 * the (k+1)-th ...: every stream keeps its own order, and all of them are fed at the same pace (a host that enqueues
 * one chain after the other starts the second one a whole chain's worth of launch calls late).  new_index (may be
 * NULL) receives, for every old node index, the node's new index. */
int32_t kxc_hip_plan_interleave_chains(kxc_hip_plan* plan, int32_t* new_index, int32_t capacity);
int32_t kxc_hip_plan_set_select_lanes(kxc_hip_plan* plan, int32_t lanes);
int32_t kxc_hip_set_select_lanes(int32_t lanes);
/* Allocate the workspace (bytes = the largest offset + size the nodes use). */
int32_t kxc_hip_plan_finalize(kxc_hip_plan* plan, size_t workspace_bytes);
/* Enqueue every node on `stream`; returns after enqueue (no synchronisation). */
int32_t kxc_hip_plan_run(kxc_hip_plan* plan, void** packed_args, void* stream);
/* HIP graph replay for launch-bound plans (batch-1 inference: ~25 launches of ~15 us).  When enabled, the second
 * run on a non-null stream is recorded by stream capture (side-lane nodes become parallel branches) and every
 * later run with the same packed-argument pointers is one hipGraphLaunch; other pointers re-capture.  The first
 * run stays eager so that lazily allocated scratch exists before the capture.  The plan records no memset node. */
int32_t kxc_hip_plan_enable_graph(kxc_hip_plan* plan, int32_t enable);
/* The same run with a HIP event between consecutive launches: fills one record per plan node (kernel symbol,
 * launch geometry, start relative to the first launch, duration) and returns after the last launch has
 * finished.  The records carry what the reference's profiler adapter puts into a "cuda_kernel" event
 * (src/base/profiling.cc:623-651: grid_x..block_z, dynamic_shared_memory, start, end); the host layer turns
 * them into component "backend.hip" events.  *count = number of nodes; fails if capacity is smaller. */
#define KXC_HIP_RECORD_KERNEL 0
#define KXC_HIP_RECORD_MEMCPY 1
typedef struct kxc_hip_launch_record {
    char kernel_symbol[120];
    int32_t kind;                    /* KXC_HIP_RECORD_* */
    uint32_t grid[3], block[3];
    uint32_t dynamic_shared_memory;
    int64_t bytes;                   /* copies only */
    int64_t start_ns, duration_ns;
} kxc_hip_launch_record;
int32_t kxc_hip_plan_run_profiled(kxc_hip_plan* plan, void** packed_args, void* stream,
                                  kxc_hip_launch_record* records, int32_t capacity, int32_t* count);
int32_t kxc_hip_plan_num_nodes(const kxc_hip_plan* plan);
/* kernel_symbol of node i (static storage owned by the plan). */
const char* kxc_hip_plan_node_symbol(const kxc_hip_plan* plan, int32_t i);
/* Device address of the workspace (NULL before finalize): lets tests read intermediates. */
void* kxc_hip_plan_workspace(const kxc_hip_plan* plan);

#ifdef __cplusplus
}
#endif
#endif  /* KXC_HIP_H_ */
