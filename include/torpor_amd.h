/* torpor_amd: C-ABI of the MI355X-native model-swapping inference engine.
 *
 * The reference server (FCSLab/torpor) has no C-ABI of its own: its wire layer
 * calls header-only C++ classes directly.  Each entry point below therefore
 * names the reference method whose job it does (paths relative to the
 * reference tree).  A ZMQ front end binds these exactly where the reference
 * dispatches a SignalRequest (include/server/controller.hpp:128-216) or a
 * WapperQuery (include/server/cuda_server.hpp:301-455).
 *
 * Conventions
 *   - return value: 0 = ok, negative = engine error (TP_E*), positive = hipError_t.
 *   - no exceptions or aborts cross this boundary.
 *   - device addresses handed to callers are opaque 64-bit *virtual* addresses
 *     that stay valid across swap-out / swap-in (the reference's
 *     cudaMallocResponse.ptr, proto/cudarpc.proto:303-306).
 *   - the caller keeps ownership of every host buffer it passes; the engine
 *     copies in and out.
 *   - one control thread and one executor thread may call concurrently; there
 *     is one active function per GPU at a time (cuda_server.hpp:1371,
 *     controller.hpp:415).
 *   - asynchronous op failures are sticky and reported by the next
 *     tp_stream_synchronize / tp_device_synchronize (same wire field as the
 *     reference's `int32 error`, proto/cudarpc.proto:85-87).
 */
#ifndef TORPOR_AMD_H
#define TORPOR_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tp_server tp_server;

/* ---- error codes (negative) ---- */
#define TP_OK 0
#define TP_EINVAL (-22)        /* bad argument / shape */
#define TP_ENOMEM (-12)        /* pool or host store exhausted */
#define TP_ENOENT (-2)         /* unknown function / address */
#define TP_EBUSY (-16)         /* executor busy or function active */
#define TP_ENODEV (-19)        /* engine created with TP_FLAG_HOST_ONLY: no compute, no device memory */
#define TP_ESTATE (-71)        /* call not valid in the executor's current mode */
#define TP_ENOTACTIVE (-72)    /* client id is not the active function */
#define TP_EUNSUPPORTED (-38)  /* shape / option not implemented */
#define TP_EFAULT (-14)        /* virtual address does not translate */
#define TP_ERANGE (-34)        /* function id above TP_MAX_FUNCTION_ID */
#define TP_ESCRATCH (-75)      /* the call needs more scratch memory than tp_gemm_noalloc's fixed buffer holds */

/* Function ids are decimal strings, as in the reference (stoi(func), cuda_server.hpp:221-224), in
 * 0 .. TP_MAX_FUNCTION_ID: the id is part of every virtual address handed to the function. */
#define TP_MAX_FUNCTION_ID 65535

/* ---- signal.proto enums (proto/signal.proto:5-30) ---- */
#define TP_REQ_EXECUTE_AFTER_LOAD 0 /* register model */
#define TP_REQ_EXECUTE 1            /* invoke */
#define TP_REQ_LOAD 2               /* swap-in (prefetch) */
#define TP_REQ_UNLOAD 3             /* swap-out */
#define TP_REQ_EXECUTE_FOR_RECORD 10
#define TP_REQ_REPLAY 11
#define TP_ACK_OK 0
#define TP_ACK_INAVAIL 1

/* ---- tp_config.flags ---- */
#define TP_FLAG_HOST_ONLY 1 /* no HIP calls: pool/LRU/state-machine logic only (CPU tests) */
#define TP_FLAG_EVICT_LRU 2 /* plain LRU eviction, as env EVICT_POLICY=LRU (controller.hpp:103-109); default: two-class */
#define TP_FLAG_NO_HOST_GATHER 4 /* embedding lookups always wait for their table's transfer group, as env TORPOR_HOST_GATHER=0 */
#define TP_FLAG_NO_PACK 8 /* weights cross the link as they are instead of in the packed transfer format, as env TORPOR_PACK=0 */
#define TP_FLAG_POOL_FIXED 32 /* pool policy of FixedSizeBlockManager, as env BLOCK_MANAGER=Fixed (memory_manager.hpp:46-52,
                               * block_manager.hpp:188-258): released extents are kept per exact size and reused, newest first */
#define TP_FLAG_KEEP_HOST_IMAGE 16 /* keep the raw weight image in pinned host memory beside the packed transfer image (by default the
                                   * transfer image, checked to decode back bit for bit, is the host store), as env TORPOR_SLIM_HOST=0 */

/* ---- activation / epilogue ---- */
#define TP_ACT_NONE 0
#define TP_ACT_RELU 1
#define TP_ACT_GELU 2 /* erf form */
#define TP_ACT_TANH 3
#define TP_ACT_RELU6 4
#define TP_ACT_SILU 5
#define TP_ACT_SIGMOID 6

/* ---- tensor layouts for convolution / pooling / batch-norm ---- */
#define TP_LAYOUT_NCHW 0
#define TP_LAYOUT_NHWC 1

/* ---- op ids for tp_launch (takes the place of launching libtorch kernels by
 *      mangled name, cuda_server.hpp:1226-1310) ----
 *   ptr / int / float argument lists per op:                                  */
#define TP_OP_RELU 1         /* p: x,y          i: n */
#define TP_OP_ADD 2          /* p: a,b,y        i: n, relu */
#define TP_OP_BIAS_ACT 3     /* p: x,bias,y     i: rows, C, act */
#define TP_OP_GELU 4         /* p: x,y          i: n */
#define TP_OP_MAXPOOL 5      /* p: x,y          i: N,H,W,C,k,stride,pad,layout[,y_pitch (NHWC, 0 = C)] */
#define TP_OP_AVGPOOL 6      /* p: x,y          i: N,HW,C,layout   (global average) */
#define TP_OP_LAYERNORM 7    /* p: x,res|0,gamma,beta,y  i: rows,width  f: eps */
#define TP_OP_SOFTMAX 8      /* p: x,mask|0,y   i: rows,width,rows_per_mask  f: scale */
#define TP_OP_EMBEDDING 9    /* p: ids,type_ids|0,word,pos|0,type|0,y  i: tokens,seq,width,vocab,n_types */
#define TP_OP_NCHW_TO_NHWC 10 /* p: x,y         i: N,C,H,W */
#define TP_OP_NHWC_TO_NCHW 11 /* p: x,y         i: N,C,H,W */
#define TP_OP_SUM 12         /* p: x,y          i: n */
#define TP_OP_FILL 13        /* p: y            i: n   f: value */
/* Fused attention, out[b,q,a,:] = softmax_k(scale * Q[b,q,a,:].K[b,k,a,:] + mask[b,k]) . V[b,k,a,:].  Row (b*S + t)
 * of q / k / v / out starts at pointer + (b*S + t)*ld floats, head a at column a*dh; mask is [B][S] additive or 0.
 * Stands in for the reference's cublasSgemmStridedBatched + softmax launch + cublasSgemmStridedBatched sequence
 * (include/server/cuda_server.hpp:524-550,1226-1310).  dh must be 64, strides multiples of 4 floats, pointers 16 B
 * aligned (TP_EUNSUPPORTED otherwise: issue the three separate calls instead). */
#define TP_OP_ATTENTION 14   /* p: q,k,v,mask|0,out  i: B,A,S,dh,ldq,ldk,ldv,ldo  f: scale */
#define TP_OP_AVGPOOL2D 15   /* p: x,y   i: N,H,W,C,k,stride,pad,y_pitch|0   NHWC window average, padding counted */
#define TP_OP_COPY2D 16      /* p: src,dst   i: rows,width,src_pitch,dst_pitch   (elements) */
#define TP_OP_SCALE_CHANNELS 17 /* p: x,scale,y   i: N,HW,C   y[n,p,c] = x[n,p,c] * scale[n,c] (NHWC) */
/* Inference batch-norm (+ ReLU) of the input, 1x1 convolution, epilogue -- one launch for what a pre-activation
 * network issues as cudnnBatchNormalizationForwardInference + activation + cudnnConvolutionForward
 * (cuda_server.hpp:797-860, 708-771).  NHWC: x is rows pixels of cin channels, x_pitch floats apart (0 = cin: the
 * first cin channels of a wider tensor otherwise); w is [cout][cin]; y rows of cout, y_pitch apart (0 = cout).
 * The four pre_* vectors [cin] normalise x -- or, with pre_beta = pre_mean = pre_var = 0, pre_gamma alone scales
 * it per channel (the gate of a squeeze-and-excitation block applied to one image); the four post_* vectors [cout]
 * (all or none), an optional residual laid out like y and `act` form the epilogue.  Taken: cin a multiple of 32 up to 2048, x / w / the vectors 16-byte aligned, x_pitch a multiple of 4;
 * TP_EUNSUPPORTED otherwise (the caller issues the two calls instead).
 *   p: x,pre_gamma,pre_beta|0,pre_mean|0,pre_var|0,w,y,post_gamma|0,post_beta|0,post_mean|0,post_var|0[,residual|0]
 *   i: rows,cin,cout,x_pitch,y_pitch,pre_relu,act   f: pre_eps,post_eps */
#define TP_OP_BN_CONV1X1 18

typedef struct tp_config {
    uint32_t struct_size;       /* sizeof(tp_config) */
    int32_t device;             /* HIP device ordinal */
    uint64_t mem_limit_bytes;   /* LRU budget; 0: env MEM_LIMIT_IN_GB or 24 GiB (controller.hpp:83-93) */
    uint64_t pool_bytes;        /* HBM arena; 0: mem_limit + pool headroom (memory_manager.hpp:42-44) */
    uint64_t chunk_bytes;       /* first swap-in gate group; 0: env BUFFER_SIZE or 2 MiB (memory_manager.hpp:22,169-173);
                                   below 256 (the reference's BUFFER_SIZE=1 ablation): one group per tensor */
    uint64_t chunk_max_bytes;   /* groups double up to this size; 0: chosen per model (16 MiB with two copy streams,
                                 * 32 MiB with one); set = chunk_bytes for fixed groups */
    uint64_t workspace_bytes;   /* split-K scratch; 0: 64 MiB */
    int32_t flags;              /* TP_FLAG_* */
    int32_t request_timeout_ms; /* 0: 5000 (cuda_server.hpp:29) */
    int32_t copy_streams;       /* swap-in copy streams: 0 = chosen per model, 1 or 2 */
    int32_t reserved0;
} tp_config;

typedef struct tp_epilogue {
    float alpha;       /* scales the accumulator */
    float beta;        /* + beta * previous C */
    uint64_t bias;     /* [N] or 0 */
    uint64_t bn_scale; /* inference batch-norm gamma [N] or 0; the four bn_* go together */
    uint64_t bn_bias;
    uint64_t bn_mean;
    uint64_t bn_var;
    float bn_eps;
    int32_t act;       /* TP_ACT_* */
    uint64_t residual; /* same shape as C, or 0 */
    int64_t ldr;       /* row pitch of residual (0: same as C) */
} tp_epilogue;

/* Row-major GEMM C[r][c] = epilogue(sum_k X(r,k) * Y(c,k)), X(r,k) at x + r*xs_r + k*xs_k
 * (elements), Y(c,k) at y + c*ys_c + k*ys_k; batch z = b0*nb1 + b1. */
typedef struct tp_gemm_desc {
    uint64_t x, y, c;
    int64_t m, n, k;
    int64_t xs_r, xs_k, ys_c, ys_k, ldc;
    int32_t nb0, nb1;
    int64_t xb0, xb1, yb0, yb1, cb0, cb1;
    tp_epilogue ep;
} tp_gemm_desc;

typedef struct tp_conv_desc {
    uint64_t x, w, y; /* w is [Cout][Cin][KH][KW] */
    int32_t n, h, w_in, cin, cout, kh, kw;
    int32_t stride_h, stride_w, pad_h, pad_w, groups;
    int32_t x_layout, y_layout; /* TP_LAYOUT_* */
    /* NHWC only: elements between consecutive pixels of x / y, 0 = cin / cout.  A larger pitch reads the first
     * cin channels of a wider tensor, or writes a channel slice of one (concatenation without a copy).
     * groups: 0 / 1; cin == cout == groups (depthwise, NHWC, w is [C][1][KH][KW]); or any divisor of cin and cout
     * (cudnnSetConvolutionGroupCount, cuda_server.hpp:671; NHWC in and out, w is [cout][cin/groups][KH][KW], one
     * launch per group). */
    int64_t x_pitch, y_pitch;
    tp_epilogue ep;
} tp_conv_desc;

typedef struct tp_pool_stats {
    uint64_t capacity, used, largest_free;
    uint64_t live_extents, free_extents;
    uint64_t lru_budget, lru_used, lru_models;
    uint64_t evictions, swap_ins;
    /* victims taken because no contiguous extent fitted although the budget test had passed (the reference
     * exits there, block_manager.hpp:345-351); they are included in `evictions` */
    uint64_t fragmentation_evictions;
    /* pinned host memory: raw weight images (whole, for models that travel as they are; only the tables looked
     * up by index for models whose packed transfer image is their host store), transfer images, request
     * staging and result buffers */
    uint64_t host_image_bytes, host_transfer_bytes, host_staging_bytes;
    /* device memory outside the pool and its budget: staging area of packed transfers, kernel workspace */
    uint64_t device_staging_bytes, device_workspace_bytes;
    /* TP_FLAG_POOL_FIXED: released extents waiting in the per-size idle lists (not part of `used`) */
    uint64_t pool_cached_bytes, pool_idle_extents;
} tp_pool_stats;

typedef struct tp_model_info {
    int32_t registered; /* host store complete */
    int32_t resident;   /* weights allocated in the pool */
    int32_t level;
    int32_t n_params;
    int32_t n_chunks;
    int32_t n_ops;       /* recorded program length */
    uint64_t image_bytes; /* weight image (256 B aligned tensors, first-access order) */
    uint64_t param_bytes; /* sum of tensor sizes */
    uint64_t act_bytes;   /* activation arena */
    uint64_t total_bytes; /* what the LRU charges */
    uint64_t weight_off;  /* pool offsets when resident */
    uint64_t act_off;
} tp_model_info;

typedef struct tp_swap_stats {
    uint64_t bytes;      /* bytes the last swap-in of this model moved over the host link (below the image size when
                            tensors travel in the packed transfer format) */
    double copy_ms;      /* first copy issued -> last group in place (landed and, if packed, expanded) */
    double alloc_us;     /* host time to (re)acquire pool extents ("CheckMalloc", memory_manager.hpp:499-501) */
    double evict_us;     /* host time of the last swap-out (memory_manager.hpp:258) */
    uint32_t chunks;
    uint32_t gate_waits; /* compute-stream waits issued during the last request */
    uint32_t copy_streams; /* streams the last swap-in alternated over */
    uint32_t host_gathers; /* lookups of the last request that read their table in place from the host store */
    uint64_t deferred_bytes; /* of `bytes`: transfer groups that hold nothing but tables looked up by index; they
                                travel last and a request does not wait for them */
    /* host side of the last swap-in: time the copy thread took to hand every group to the streams, and its
     * slowest single runtime call (group index; kind 0 = copy, 1 = event record, 2 = stream wait, 3 = expansion
     * launch).  A swap-in is paced by the link unless a call here stalls. */
    double issue_ms;
    double max_call_us;
    uint32_t max_call_group;
    uint32_t max_call_kind;
} tp_swap_stats;

/* ------------------------------------------------------------------ lifecycle
 * Controller ctor + CUDAExecutor::start (controller.hpp:54-121, cuda_server.hpp:92-118,
 * memory_manager.hpp:168-193, block_manager.hpp:264-273). */
int tp_server_create(const tp_config* cfg, tp_server** out);
void tp_server_destroy(tp_server* s);
const char* tp_strerror(int code);
const char* tp_version(void);

/* ------------------------------------------------------------------ control plane
 * One SignalRequest -> SignalAck exchange (controller.hpp:131-216).  `function` is the
 * decimal client id.  When the executor is busy the request is queued
 * (controller.hpp:156,177) and *deferred is set to 1: its ack appears later through
 * tp_take_deferred_ack, after the active request completes (controller.hpp:242-262).
 * Load and Unload are served while a request runs (controller.hpp:187-215); the function that is
 * running is never the victim of the eviction a Load causes, and a function whose last request is
 * still executing on the device (a request ends, for the controller, when its result copy is
 * queued: cuda_server.hpp:1044) is swapped out only after the device has finished that work. */
int tp_signal(tp_server* s, int32_t type, const char* function, const char* payload, int32_t* ack, int32_t* resp,
              int32_t* deferred);
int tp_take_deferred_ack(tp_server* s, int32_t* ack, int32_t* resp); /* 1 = ack produced, 0 = none */
/* The same two calls for a front end with many peers.  A queued signal gets a ticket (numbered from 1 in the
 * order of queueing; 0 when the signal was answered at once) and its ack comes back with that ticket, so
 * acks are matched to peers by ticket, not by position.  When the peer of a queued signal disconnects
 * (the reference's REP socket simply loses the reply, controller.hpp:433-441, and the executor then sits
 * in the orphaned request until the timeout of cuda_server.hpp:257-264) the front end cancels the ticket:
 * 1 = it was still queued and is dropped, no ack will appear; 2 = its request had been started meanwhile:
 * the pending ack is dropped and the request is completed at once (a half-finished registration is
 * forgotten); 0 = unknown ticket or ack already taken. */
int tp_signal_ticket(tp_server* s, int32_t type, const char* function, const char* payload, int32_t* ack,
                     int32_t* resp, int32_t* deferred, uint64_t* ticket);
int tp_take_deferred_ack_ticket(tp_server* s, int32_t* ack, int32_t* resp, uint64_t* ticket);
int tp_cancel_deferred(tp_server* s, uint64_t ticket);
/* Request-timeout check of the executor loop (cuda_server.hpp:257-264); returns 1 when a
 * timed-out request was force-completed. */
int tp_poll(tp_server* s);

/* ------------------------------------------------------------------ data plane: memory
 * cudaMallocService / cudaFreeService (cuda_server.hpp:965-992, memory_manager.hpp:85-110). */
int tp_malloc(tp_server* s, int32_t client, uint64_t bytes, uint64_t* vaddr);
int tp_free(tp_server* s, int32_t client, uint64_t vaddr);
/* 0 when [vaddr, vaddr + bytes) lies inside one block that the active function `client` may address now;
 * no side effects.  For a front end that must set aside `bytes` of its own before the copy is validated
 * (the reference mallocs `count` bytes unchecked, cuda_server.hpp:1007,1040). */
int tp_check_address(tp_server* s, int32_t client, uint64_t vaddr, uint64_t bytes);
/* cudaMemcpyService / cudaMemcpyAsyncService H2D (cuda_server.hpp:994-1037); while the
 * function is being registered the bytes go to the host weight store
 * (memory_manager.hpp:124-142, model_repo.hpp:151-168). */
int tp_memcpy_h2d(tp_server* s, int32_t client, uint64_t dst, const void* src, uint64_t bytes);
/* cudaMemcpyAsyncService D2H (cuda_server.hpp:1038-1045): staged, delivered into `dst` by the
 * next tp_stream_synchronize, and marks the request finished (send_complete_signal). */
int tp_memcpy_d2h_async(tp_server* s, int32_t client, void* dst, uint64_t src, uint64_t bytes);
/* cudaMemcpyService D2H (cuda_server.hpp:1006-1011): synchronous, no completion side effect. */
int tp_memcpy_d2h(tp_server* s, int32_t client, void* dst, uint64_t src, uint64_t bytes);
int tp_memcpy_d2d(tp_server* s, int32_t client, uint64_t dst, uint64_t src, uint64_t bytes); /* cuda_server.hpp:1047-1051 */
int tp_memset_async(tp_server* s, int32_t client, uint64_t dst, int32_t value, uint64_t bytes); /* cuda_server.hpp:1058-1068 */
/* cudaDeviceSynchronizeService (cuda_server.hpp:951-962): also ends the weight-upload phase of a
 * registration and starts access tracking. */
int tp_device_synchronize(tp_server* s, int32_t client);
/* cudaStreamSynchronizeService (cuda_server.hpp:1132-1149). */
int tp_stream_synchronize(tp_server* s, int32_t client);

/* ------------------------------------------------------------------ data plane: compute */
/* cublasSgemmService (cuda_server.hpp:502-522): column-major, op(A) m x k, op(B) k x n.
 * transa/transb: 0 = N, 1 = T. */
int tp_sgemm(tp_server* s, int32_t client, int32_t transa, int32_t transb, int32_t m, int32_t n, int32_t k,
             float alpha, uint64_t a, int32_t lda, uint64_t b, int32_t ldb, float beta, uint64_t c, int32_t ldc);
/* cublasSgemmStridedBatchedService (cuda_server.hpp:524-550). */
int tp_sgemm_strided_batched(tp_server* s, int32_t client, int32_t transa, int32_t transb, int32_t m, int32_t n,
                             int32_t k, float alpha, uint64_t a, int32_t lda, int64_t stride_a, uint64_t b,
                             int32_t ldb, int64_t stride_b, float beta, uint64_t c, int32_t ldc, int64_t stride_c,
                             int32_t count);
/* Row-major GEMM with fused epilogue and two-level batching (the HIP-native form of the two above). */
int tp_gemm(tp_server* s, int32_t client, const tp_gemm_desc* d);
/* cudnnConvolutionForwardService (cuda_server.hpp:708-735), shapes inline instead of descriptor
 * handles (cuda_server.hpp:579-706), optional fused epilogue. */
int tp_conv_forward(tp_server* s, int32_t client, const tp_conv_desc* d);
/* cudnnBatchNormalizationForwardInferenceService (cuda_server.hpp:737-771). */
int tp_bn_inference(tp_server* s, int32_t client, uint64_t x, uint64_t y, uint64_t scale, uint64_t bias,
                    uint64_t mean, uint64_t var, double eps, int64_t rows, int32_t channels, int64_t hw,
                    int32_t layout, int32_t relu);
/* The same with rows of x `x_pitch` elements apart (NHWC; 0 = channels): normalises the first `channels`
 * channels of a wider tensor into a dense y. */
int tp_bn_inference_pitched(tp_server* s, int32_t client, uint64_t x, uint64_t y, uint64_t scale, uint64_t bias,
                            uint64_t mean, uint64_t var, double eps, int64_t rows, int32_t channels, int64_t hw,
                            int32_t layout, int32_t relu, int64_t x_pitch);
/* tp_gemm for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference.  The descriptor is tp_gemm's, except
 * that x / y / c and the epilogue's pointers are raw device addresses on the current HIP device (not an
 * engine's virtual addresses) and the work is enqueued on `stream` (a hipStream_t; NULL = the default
 * stream); no tp_server is involved.  The call allocates nothing on host or device: the partial sums of
 * a GEMM whose K range is split over workgroups go to a fixed TP_NOALLOC_SCRATCH_BYTES array that each
 * GPU the library runs on holds until the process ends.  Results are bit-identical to tp_gemm's.
 *   - a shape whose partial sums need more than that array is refused with TP_ESCRATCH (a split happens for
 *     fewer 64x64 output tiles than CUs, so m * n <= 1 Mi elements with at most 32 slots, or as a pair of K
 *     halves for up to three tiles per CU when both halves fit the array);
 *   - all calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads)
 *     race on it.  Calls on one stream are ordered and safe.
 *   - the first call on each GPU looks up that GPU's copy of the array and the device's properties, which
 *     may load the library's code object: make it before the stretch in which nothing may be allocated
 *     (outside graph capture); every later call on that GPU only launches.
 *   - the array's first 4 KiB are per-tile counters that are zero between launches (the workgroup that
 *     finishes a split tile last sets its counter back).  A launch that never completes (a stream destroyed
 *     under it, a device reset) leaves them undefined, and later split GEMMs on that GPU would sum wrongly:
 *     after such an event the process must not go on using this entry point. */
#define TP_NOALLOC_SCRATCH_BYTES (16u << 20)
int tp_gemm_noalloc(const tp_gemm_desc* d, void* stream);
/* cudaLaunchKernelService (cuda_server.hpp:1226-1310) by op id, pointer slots explicit. */
int tp_launch(tp_server* s, int32_t client, int32_t op_id, const uint64_t* ptrs, int32_t n_ptrs,
              const int64_t* ints, int32_t n_ints, const float* floats, int32_t n_floats);

/* ------------------------------------------------------------------ replay
 * The op stream of the first (tracked) inference is kept per function
 * (signal.proto ExecuteForRecord / Replay).  tp_replay re-issues it: recorded H2D copies read
 * consecutive slices of `input`, recorded D2H copies fill consecutive slices of `output`; it
 * includes the final stream synchronisation and completion signal. */
int tp_replay(tp_server* s, int32_t client, const void* input, uint64_t input_bytes, void* output,
              uint64_t output_bytes);
/* Optional: pinned host memory for request inputs and results.  A device-to-host copy (tp_memcpy_d2h_async, or
 * tp_replay's `output`) whose destination lies inside such a buffer is written there by the device
 * directly; any other destination is filled through the engine's pinned staging buffer and one host copy
 * after the stream synchronisation.  A host-to-device copy (tp_memcpy_h2d, or tp_replay's `input`) whose
 * source lies inside such a buffer is read by the device where it lies -- the caller leaves it unchanged
 * until the next synchronising call of that function (tp_stream_synchronize, or tp_replay returning), as with
 * any asynchronous copy from pinned memory; any other source is copied into the engine's staging buffer
 * before the call returns and may be reused at once.  No counterpart in the reference, whose clients pass
 * inputs and receive results through the shared-memory segment they registered (cuda_server.hpp:1030-1046).
 * Buffers are released by tp_host_free or with the server. */
int tp_host_alloc(tp_server* s, uint64_t bytes, void** ptr);
int tp_host_free(tp_server* s, void* ptr);

/* ------------------------------------------------------------------ introspection (tests, bench) */
int tp_model_resident(tp_server* s, int32_t client); /* 1/0, negative on error */
/* 1 when the function is resident and every transfer group of its last swap-in is in place, 0 while a swap-in is
 * still on its way or the function is swapped out (asked of the device without waiting).  The reference keeps this
 * per tensor in ParamLocMap (memory_manager.hpp:33,590) and never exposes it. */
int tp_model_loaded(tp_server* s, int32_t client);
/* What a scheduler above the boundary needs in order to place a request of a swapped-out function: how long the
 * swap-in occupies the host link before the request can complete (bytes the request waits for / the link rate the
 * engine measured), and the forward pass as it runs beside that swap-in (timed at registration, the best warm
 * request since, plus what active copy queues cost each launch).  The
 * reference's router and simulator work from per-model constants instead (scripts/router.py:17,
 * misc/tools/node_simu.py:99-117). */
int tp_get_load_estimate(tp_server* s, int32_t client, double* swap_ms, double* forward_ms);
int tp_get_model_info(tp_server* s, int32_t client, tp_model_info* out);
int tp_get_pool_stats(tp_server* s, tp_pool_stats* out);
int tp_get_swap_stats(tp_server* s, int32_t client, tp_swap_stats* out);
/* Copies the device-resident weight image (waits for an in-flight swap-in). */
int tp_readback_weights(tp_server* s, int32_t client, void* dst, uint64_t bytes);
/* The authoritative host copy of the same image, same layout.  For a model whose host store is its packed
 * transfer image the image is decoded into a buffer of the engine's; *ptr stays valid until the next
 * tp_host_weights call on this server (or the server's destruction). */
int tp_host_weights(tp_server* s, int32_t client, const void** ptr, uint64_t* bytes);
/* Image offset of a weight virtual address (first-access-order layout). */
int tp_weight_offset(tp_server* s, int32_t client, uint64_t vaddr, uint64_t* image_off);
/* Name of the kernel variant chosen by the last compute op on the calling thread. */
const char* tp_last_kernel(void);
/* Pinned-host -> HBM link probe: one hipMemcpyAsync of `bytes`, median of `iters`; GB/s. */
int tp_measure_h2d(tp_server* s, uint64_t bytes, int32_t iters, double* gbps);
/* Runs `iters` timed repetitions of the last compute op recorded for `client` at program index
 * `op_index` (or -1: last op) and returns the mean duration in microseconds measured with HIP
 * events on the compute stream. */
int tp_time_op(tp_server* s, int32_t client, int32_t op_index, int32_t iters, double* mean_us);

/* Per-kernel timing of the compute stream, for roofline accounting.  Between begin and end
 * every compute op is bracketed by two HIP events on the compute stream; end waits for the
 * stream and aggregates by kernel variant.  tp_profile_read returns TP_ENOENT past the last
 * entry.  The entry named "__empty_bracket__" is the duration of an empty bracket (event
 * overhead), measured at end, to be subtracted per launch.  No counterpart in the reference,
 * which logs host-side timestamps only (memory_manager.hpp:425-431, cuda_server.hpp:294-295). */
typedef struct tp_kernel_stat {
    char name[64];   /* kernel variant; GEMM and convolution launches carry their shape: name[MxNxK] or
                        name[NxHxWxCin>Cout kKHxKW sS] */
    uint64_t launches;
    double total_us; /* sum of bracketed durations */
    double flops;    /* algorithmic floating-point operations of those launches */
    double bytes;    /* algorithmic bytes read + written */
} tp_kernel_stat;
int tp_profile_begin(tp_server* s);
int tp_profile_end(tp_server* s);
int tp_profile_read(tp_server* s, int32_t index, tp_kernel_stat* out);

/* ------------------------------------------------------------------ host-side building blocks
 * The pool allocator and the eviction policy as stand-alone objects (pure host logic, no device),
 * so that they can be unit-tested and reused by a front end.
 * tp_pool: extents of 2 MiB slabs out of one arena, best fit, coalescing; takes the place of
 *          BuddyBasedBlockManager (block_manager.hpp:260-418).  Offsets are arena-relative;
 *          UINT64_MAX = no fit.
 * tp_lru:  LRUEvictor (evictor.hpp:190-264).  check_and_add writes the victims, oldest first and
 *          newline-separated, into `victims` (truncated to `cap` bytes incl. the terminator). */
typedef struct tp_pool tp_pool;
#define TP_POOL_BEST_FIT 0   /* default */
#define TP_POOL_FIXED_SIZE 1 /* FixedSizeBlockManager (block_manager.hpp:188-258): per-size idle lists, newest first;
                              * idle extents are given back, largest size first, when a new size does not fit */
tp_pool* tp_pool_create(uint64_t capacity_bytes);
tp_pool* tp_pool_create_policy(uint64_t capacity_bytes, int32_t policy);
/* fixed-size policy: bytes and count of idle extents; tp_pool_trim gives them all back and returns the count */
int tp_pool_cached(tp_pool* p, uint64_t* cached_bytes, uint64_t* idle_extents);
int tp_pool_trim(tp_pool* p);
void tp_pool_destroy(tp_pool* p);
uint64_t tp_pool_alloc(tp_pool* p, uint64_t bytes);
int tp_pool_release(tp_pool* p, uint64_t offset);
int tp_pool_query(tp_pool* p, uint64_t* capacity, uint64_t* used, uint64_t* largest_free, uint64_t* live_extents,
                  uint64_t* free_extents);
typedef struct tp_lru tp_lru;
tp_lru* tp_lru_create(uint64_t budget_bytes);
void tp_lru_destroy(tp_lru* l);
int tp_lru_check_and_add(tp_lru* l, const char* function, uint64_t size, char* victims, uint64_t cap,
                         int32_t* n_victims, int32_t* over_budget);
int tp_lru_force_evict(tp_lru* l, const char* function); /* 1 = was tracked, 0 = unknown */
int tp_lru_lock(tp_lru* l, const char* function);
int tp_lru_unlock(tp_lru* l, const char* function);
uint64_t tp_lru_used(tp_lru* l);

/* Control-plane policy objects for a node with several GPUs; decision logic only, no device calls.
 * tp_evictor: the Evictor interface (evictor.hpp:14-26) with one budget per GPU.  TP_EVICT_LRU is LRUEvictor
 *             (evictor.hpp:190-264); TP_EVICT_IA is InterferenceAwareEvictor (evictor.hpp:28-188): models of level
 *             >= 1 that only one GPU holds are evicted after everything else.  Levels are those of the
 *             ExecuteAfterLoad payload (controller.hpp:142-152), 0 light / 1 median / 2 heavy, default 0.
 *             check_and_add writes victims as tp_lru_check_and_add does; order() writes the eviction order of one
 *             GPU, first victim first.
 * tp_sched:   executor states, residency and link tables of the controller, and its three decisions:
 *             placement() (controller.hpp:271-294), TP_SCHED_RANDOM (controller.hpp:296-319) and TP_SCHED_IA
 *             (controller.hpp:321-389).  status values are the reference's ExecutorStatus (-1 idle, 0 local, 1 peer
 *             copy, 2..4 host-link swap of a light / median / heavy model, 5 cold start).  `draw` replaces rand()
 *             of the random policy so that callers (and tests) own the random stream.  decide() returns 0 and
 *             dst = -1 when no executor is idle.
 * Neither object locks: the reference calls its evictor and scheduler from the controller thread only
 * (controller.hpp:128-216), and so must a caller of these. */
#define TP_EVICT_LRU 0
#define TP_EVICT_IA 1
typedef struct tp_evictor tp_evictor;
tp_evictor* tp_evictor_create(int32_t policy, int32_t gpu_count, uint64_t budget_bytes);
void tp_evictor_destroy(tp_evictor* e);
int tp_evictor_set_level(tp_evictor* e, const char* function, int32_t level);
int tp_evictor_check_and_add(tp_evictor* e, int32_t gpu, const char* function, uint64_t size, char* victims,
                             uint64_t cap, int32_t* n_victims, int32_t* over_budget);
int tp_evictor_force_evict(tp_evictor* e, int32_t gpu, const char* function); /* 1 = was tracked */
int tp_evictor_lock(tp_evictor* e, int32_t gpu, const char* function);
int tp_evictor_unlock(tp_evictor* e, int32_t gpu, const char* function);
uint64_t tp_evictor_used(tp_evictor* e, int32_t gpu);
int tp_evictor_is_protected(tp_evictor* e, int32_t gpu, const char* function); /* TP_EVICT_IA: 1 = evicted last */
int tp_evictor_order(tp_evictor* e, int32_t gpu, char* out, uint64_t cap);

#define TP_SCHED_RANDOM 0
#define TP_SCHED_IA 1
typedef struct tp_sched tp_sched;
tp_sched* tp_sched_create(int32_t gpu_count);
void tp_sched_destroy(tp_sched* s);
int tp_sched_set_sibling(tp_sched* s, int32_t gpu, int32_t other); /* shares the host link (PCIe switch) */
int tp_sched_set_link(tp_sched* s, int32_t a, int32_t b, int32_t kind); /* -1 none, 0 self, 1 slow, 2 fast */
int tp_sched_set_status(tp_sched* s, int32_t gpu, int32_t status);
int tp_sched_set_level(tp_sched* s, const char* function, int32_t level);
int tp_sched_set_resident(tp_sched* s, const char* function, int32_t gpu, int32_t resident);
int tp_sched_placement(tp_sched* s); /* GPU for a cold start, -1 if none idle */
int tp_sched_decide(tp_sched* s, int32_t policy, const char* function, uint32_t draw, int32_t* dst_gpu,
                    int32_t* src_gpu, int32_t* status);

/* ------------------------------------------------------------------ transfer format
 * The lossless format in which compressible weight tensors cross the host link (TP_FLAG_NO_PACK
 * switches it off); no counterpart in the reference, which sends weights as they are
 * (memory_manager.hpp:378-409).  A tensor is n 32-bit words of any content.
 *   payload: units of 64 words in 216 bytes -- eight groups of eight 24-bit little-endian fields
 *            (sign << 23 | mantissa), then 24 bytes of exponent codes: group g of the unit in bits
 *            24g..24g+23, word j of the group in bits 3j..3j+2 of those.  Code c < 7 stands for
 *            exponent base + c, code 7 for "next byte of the extension stream".  The last unit is
 *            padded with zero words (code 0).
 *   extension stream: the exponent bytes of the words with code 7, in word order.
 *   block table: entry b = number of extension bytes that belong to words before word 2048 b
 *            (the device expands blocks of 2048 words independently).
 * Exposed so that the format can be checked on the host and the device kernel on its own; the engine
 * applies it by itself.
 *   tp_pack_bound / tp_pack_blocks   payload bytes / block-table entries for n words
 *   tp_pack_words    chooses the window of 7 exponents that holds the most words and packs; returns
 *                    TP_ENOMEM when the extension stream needs more than ext_cap bytes (*n_ext still
 *                    holds the count)
 *   tp_unpack_words  the inverse on the host
 *   tp_unpack_words_device  the inverse by the kernel a swap-in uses (through the engine's workspace,
 *                    synchronous), for words [w_from, w_to) only -- w_from a multiple of 64, w_to a
 *                    multiple of 64 or n_words -- as for a transfer group that ends inside a tensor;
 *                    the other words come back as 0xA5A5A5A5.  TP_EINVAL when it does not fit the
 *                    workspace. */
uint64_t tp_pack_bound(uint64_t n_words);
uint64_t tp_pack_blocks(uint64_t n_words);
int tp_pack_words(const uint32_t* words, uint64_t n_words, uint8_t* payload, int32_t* base, uint8_t* ext,
                  uint64_t ext_cap, uint64_t* n_ext, uint32_t* block_tab);
int tp_unpack_words(const uint8_t* payload, uint64_t n_words, int32_t base, const uint8_t* ext, uint64_t n_ext,
                    uint32_t* words);
int tp_unpack_words_device(tp_server* s, const uint8_t* payload, uint64_t n_words, int32_t base, const uint8_t* ext,
                           uint64_t n_ext, const uint32_t* block_tab, uint64_t w_from, uint64_t w_to,
                           uint32_t* words);

#ifdef __cplusplus
}
#endif
#endif /* TORPOR_AMD_H */
