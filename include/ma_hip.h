/*
 * ma_hip.h - C ABI of libma_hip.so: the MonarchAttention forward pass on one
 * MI355X (gfx950), hand-written HIP kernels.
 *
 * This is the boundary a host binding attaches to.  It replaces the body of
 * the reference's implementation function
 *
 *     monarch_attention_torch(q, k, v, attn_mask, T, B, pre_pad) -> Tensor
 *         (ma/ma_torch.py:65-108; registered through register_impl,
 *          ma/monarch_attention.py:15-22, called from
 *          MonarchAttention.forward, ma/monarch_attention.py:50-59)
 *
 * Plain pointers and sizes only: no torch types, no C++ in the signatures.
 * The library never allocates, frees or synchronises device memory in the
 * entry points below; every buffer belongs to the caller and all work is
 * enqueued on the stream that is passed in.  Return value of every int
 * function: 0 = ok, < 0 = ma_status, > 0 = hipError_t of a failed launch.
 *
 * Tensor conventions (the reference's, ma/ma_torch.py:74-90):
 *   q, k : (E, H, N, D)   v : (E, H, N, Dv)   out : (E, H, N, Dv) in v's dtype
 *   mask : (E, N), non-zero = keep the key/query token (see ma_mask_dtype), or NULL
 *   B block size, M = ceil(N / B) blocks, Np = M * B; zero padding at the
 *   front (pre_pad != 0) or the back; T alternating steps.
 * Strides are in ELEMENTS for the dims (e, h, n); the innermost dim must be
 * contiguous (stride 1).
 */
#ifndef MA_HIP_H_
#define MA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MA_ABI_VERSION 2

typedef enum ma_dtype { MA_F32 = 0, MA_F16 = 1, MA_BF16 = 2 } ma_dtype;

/* Element type of the (E, N) mask.  The reference combines the mask with
 * torch.logical_and (ma/ma_torch.py:98): any non-zero element keeps the token
 * (for floating-point masks -0.0 is zero and NaN is non-zero).  Callers pass bool
 * masks (its tests), int64 tokenizer masks (experiments/roberta/model.py:104-106) and
 * float 1.0 / 0.0 masks (experiments/bart/model.py:145-147); the kernels read all of
 * them in place.  mask_stride is in elements of this type. */
typedef enum ma_mask_dtype {
    MA_MASK_U8 = 0,   /* bool / uint8 / int8 */
    MA_MASK_I16 = 1,
    MA_MASK_I32 = 2,
    MA_MASK_I64 = 3,
    MA_MASK_F16 = 4,
    MA_MASK_BF16 = 5,
    MA_MASK_F32 = 6,
    MA_MASK_F64 = 7
} ma_mask_dtype;

typedef enum ma_variant {
    MA_VARIANT_AUTO = 0,    /* fastest variant that supports the problem and needs  */
                            /* nothing of the rest of the device: FUSED is chosen    */
                            /* only for callers that pass MA_FLAG_DEVICE_EXCLUSIVE,  */
                            /* everybody else gets CHAINED or STAGED in its place    */
    MA_VARIANT_GENERIC = 1, /* FMA kernels, 2T(+T-1) launches: any dtype/shape/stride */
    MA_VARIANT_STAGED = 2,  /* MFMA kernels, one launch per half step (2T launches); */
                            /* 16-bit: blocks and block counts of up to 256 rows     */
                            /* (heads of up to 65536 tokens), the one-launch         */
                            /* variants below stop at 128                            */
    MA_VARIANT_FUSED = 3,   /* MFMA, all T steps in ONE launch, teams of workgroups  */
                            /* per head, state exchanged through the workspace.  Its */
                            /* workgroups wait for each other, so the grid is sized  */
                            /* to what the device holds at once when idle: a kernel  */
                            /* of another stream or process that occupies compute    */
                            /* units for longer than the bounded waits (2^18 polls   */
                            /* of the flag a workgroup waits for, 0.1 - 0.5 s) makes */
                            /* the call fail loudly (NaN rows + error word).  Only   */
                            /* for callers that own the device while the call runs   */
    MA_VARIANT_RESIDENT = 4,/* MFMA, ONE launch, a workgroup runs whole heads with   */
                            /* the per-head state resident in LDS: with Q, K, V      */
                            /* beside it for heads of up to ~256 tokens at d = 64,   */
                            /* with one input tile at a time up to ~540, with the    */
                            /* inputs streamed (and Y through the workspace) up to   */
                            /* ~1000; several narrow workgroups per compute unit     */
                            /* when there are more short heads than compute units    */
    MA_VARIANT_CHAINED = 5  /* MFMA, ONE launch, one workgroup per block problem of  */
                            /* every phase; a problem starts when its head's         */
                            /* previous phase has released it through the workspace. */
                            /* Producers are always dispatched before consumers: no  */
                            /* co-residency requirement, safe beside other kernels   */
} ma_variant;

typedef enum ma_status {
    MA_OK = 0,
    MA_ERR_NULL = -1,        /* a required pointer is NULL                        */
    MA_ERR_SHAPE = -2,       /* a dimension, B or T is < 1 (or overflows int32)   */
    MA_ERR_DTYPE = -3,       /* unknown ma_dtype                                  */
    MA_ERR_STRIDE = -4,      /* a stride is < 0 or rows overlap                   */
    MA_ERR_WORKSPACE = -5,   /* workspace missing, misaligned or too small        */
    MA_ERR_UNSUPPORTED = -6, /* the requested variant cannot run this problem     */
    MA_ERR_VARIANT = -7,     /* unknown ma_variant                                */
    MA_ERR_DEVICE = -8,      /* no usable gfx950 device / device query failed     */
    MA_ERR_STATIC_LIMIT = -9,/* ma_fwd_static: state beyond the built-in scratch  */
    MA_ERR_BUSY = -10        /* ma_fwd_static: the scratch is still in use by a   */
                             /* call on another stream                            */
} ma_status;

/* ma_fwd_params.flags.  MA_FLAG_SYNC_READY: the caller guarantees that the sync
 * area of the workspace is zero - true after ma_workspace_init() and after every
 * completed ma_fwd() on that workspace (the one-launch kernels leave it usable).
 * Without the flag the FUSED and CHAINED variants clear the area with one extra small
 * launch in front of the forward kernel. */
#define MA_FLAG_SYNC_READY 1
/* MA_FLAG_TEST_NO_SPIN: every wait between workgroups of the one-launch variants gives
 * up at once, without looking at what it waits for.  For tests of the failure path: the call then
 * reports through the sticky error word and NaN output rows exactly as a wait that ran
 * out of time would, every kernel still runs to its end, and the next call on the
 * workspace is a normal one. */
#define MA_FLAG_TEST_NO_SPIN 2
/* MA_FLAG_DEVICE_EXCLUSIVE: the caller states that nothing else - no other stream, thread
 * or process - competes for the device's compute units while this call runs.  Only then
 * does MA_VARIANT_AUTO choose MA_VARIANT_FUSED, whose workgroups have to be on the device
 * together (on the metric workload it is 10 - 15 % ahead of CHAINED).  Setting the
 * environment variable MA_HIP_DEVICE_EXCLUSIVE=1 has the same effect for every call of the
 * process.  Without either, AUTO stays with kernels that make progress beside any other
 * work (CHAINED, RESIDENT, STAGED, GENERIC).  An explicit MA_VARIANT_FUSED is not affected. */
#define MA_FLAG_DEVICE_EXCLUSIVE 4

/* Arguments of one forward call; replaces the argument list of
 * monarch_attention_torch (ma/ma_torch.py:65-73). */
typedef struct ma_fwd_params {
    const void* q;           /* device pointers                                   */
    const void* k;
    const void* v;
    const void* mask;        /* (E, N) of mask_dtype, or NULL (ma/ma_torch.py:96-98) */
    void* out;               /* (E, H, N, Dv), dtype_v                            */
    void* workspace;         /* >= ma_fwd_workspace_bytes(), 256-byte aligned     */
    uint64_t workspace_bytes;
    int32_t E, H, N, D, Dv;
    int32_t B;               /* block size  (reference argument B)               */
    int32_t T;               /* num_steps   (reference argument T)               */
    int32_t pre_pad;         /* pad at the front instead of the back             */
    int32_t dtype_qk;        /* ma_dtype of q and k                              */
    int32_t dtype_v;         /* ma_dtype of v and out                            */
    int32_t variant;         /* ma_variant                                       */
    int32_t flags;           /* MA_FLAG_* bits, 0 if unsure                      */
    int64_t q_stride[3];     /* element strides of (e, h, n)                     */
    int64_t k_stride[3];
    int64_t v_stride[3];
    int64_t out_stride[3];
    int64_t mask_stride[2];  /* element strides of (e, n)                        */
    float eps;               /* 1e-12 in the reference (ma/ma_torch.py:10,38)    */
    int32_t mask_dtype;      /* ma_mask_dtype of the mask's elements (0 = bytes)   */
    uint32_t* error_word;    /* NULL, or a 32-bit word in pinned host memory the   */
                             /* device can write (hipHostMalloc), zero before the  */
                             /* call: a one-launch kernel whose wait runs out      */
                             /* stores the code of the sticky error word (see      */
                             /* ma_ws_layout) here as well, so that the host can    */
                             /* look at it without a copy or a synchronisation of  */
                             /* its own once the call's work is complete           */
} ma_fwd_params;

/* Byte offsets of the per-call state inside the workspace.  The arrays have
 * exactly the shapes and element types of the reference's intermediates
 * (ma/ma_torch.py:88-104), so a stage can be checked on its own:
 *   aR (E,H,M,B,D) dtype_qk   cR (E,H,M,B) f32   [inputs of the R step]
 *   aL (E,H,B,M,D) dtype_qk   cL (E,H,B,M) f32   Y (E,H,B,M,Dv) dtype_v
 *   stats: scratch of the generic L step; sync: flags of the one-launch kernels,
 *   always at offset 0 so that it does not move when one workspace serves
 *   calls of different shapes.  Its 32-bit word 1 (byte offset sync + 4) is a
 *   sticky error word a caller may read after synchronising: 0 = ok, 1 = a
 *   bounded wait between workgroups ran out (that call's output is invalid),
 *   2 = the CHAINED kernel met a producer on another XCD than its consumer. */
typedef struct ma_ws_layout {
    uint64_t aR, cR, aL, cL, Y, stats, sync, total;
} ma_ws_layout;

int ma_abi_version(void);
const char* ma_strerror(int status);

/* Validates the problem (pointers may be NULL here) and reports the workspace
 * it needs.  ma_fwd_workspace_bytes returns 0 for an invalid problem. */
int ma_fwd_workspace_layout(const ma_fwd_params* p, ma_ws_layout* layout);
uint64_t ma_fwd_workspace_bytes(const ma_fwd_params* p);

/* Zero-fills the sync area of p->workspace (one small fill kernel on `stream`);
 * afterwards calls on that workspace may pass MA_FLAG_SYNC_READY.  The
 * workspace is used by one forward call at a time: calls that share a
 * workspace must be ordered on one stream.  No counterpart in the reference
 * (its intermediates are ordinary tensors, ma/ma_torch.py:100-104). */
int ma_workspace_init(const ma_fwd_params* p, void* stream);

/* The variant MA_VARIANT_AUTO resolves to for this problem (a ma_variant), or
 * a negative ma_status. */
int ma_fwd_select_variant(const ma_fwd_params* p);

/* Name of the kernel that does the bulk of the work for this problem under the variant it resolves to
 * (for the per-stage variants: the R-step kernel), as it appears in a profiler's kernel list; NULL for an
 * invalid problem.  Introspection for benchmarks and profiles; no counterpart in the reference. */
const char* ma_fwd_kernel_name(const ma_fwd_params* p);

/* Whole forward pass: replaces monarch_attention_torch (ma/ma_torch.py:65-108).
 * `stream` is a hipStream_t (NULL = the default stream). */
int ma_fwd(const ma_fwd_params* p, void* stream);

/* ma_fwd for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose intermediates are tensors PyTorch
 * allocates, ma/ma_torch.py:88-104).  The per-call state lives in an array the
 * library itself holds on every GPU it runs on (MA_STATIC_WORKSPACE_BYTES per
 * GPU until the process ends); p->workspace, p->workspace_bytes and
 * MA_FLAG_SYNC_READY are ignored, everything else is as for ma_fwd and the
 * results are the same.  Problems whose ma_fwd_workspace_bytes() exceeds
 * MA_STATIC_WORKSPACE_BYTES return MA_ERR_STATIC_LIMIT and launch nothing (the
 * metric workload, fp16 E=1 H=16 N=4096 D=64, needs 26.8 MiB).  No device memory
 * is allocated or freed.  All calls on one GPU share that GPU's array: calls that
 * overlap in time on one GPU (different streams or threads) race.  The library
 * guards against the common case: a call on another stream than the previous
 * call's, made while that call's work has not completed, returns MA_ERR_BUSY and
 * launches nothing (calls on one stream are ordered and always accepted; streams
 * that the caller orders with events must still not have a call in flight when the
 * next is made - give such callers a workspace each through ma_fwd).  Under stream
 * capture the guard is off: replays of a captured call cannot be seen by it.  The
 * first call on a device looks up the array's address and creates the guard's event
 * (not stream operations: make one call before capturing a graph). */
#define MA_STATIC_WORKSPACE_BYTES (32u << 20)
int ma_fwd_static(const ma_fwd_params* p, void* stream);

/* One stage on the state held in the workspace (stage-level parity tests;
 * variants GENERIC and STAGED; MA_ERR_UNSUPPORTED for FUSED, RESIDENT and
 * CHAINED, whose stages are phases of a single kernel).
 *   ma_r_step  replaces al_cl_ref (ma/ma_torch.py:10-23) and, with with_v != 0,
 *              al_y_cl_ref (:38-52).  first != 0: take aR = Q, cR = 1 straight
 *              from q (the state before the first step, :88-89) instead of the
 *              workspace.  Writes aL, cL (and Y).
 *   ma_l_step  replaces ar_cr_ref (:26-35): reads aL, cL, writes aR, cR.
 *   ma_z_step  replaces z_ref (:55-62) and the final slice (:106-108): reads
 *              aL, cL, Y, writes the N real rows of out. */
int ma_r_step(const ma_fwd_params* p, int first, int with_v, void* stream);
int ma_l_step(const ma_fwd_params* p, void* stream);
int ma_z_step(const ma_fwd_params* p, void* stream);

/* Dense attention matrix: replaces MonarchAttention.get_matrix
 * (ma/monarch_attention.py:61-66), which runs the forward pass on an fp32
 * identity.  The same T steps run on q, k and the mask, then every entry
 * A[(l,j),(k,i)] = Lz[j][l,k] * R[k][j,i] is written once, in fp32: no N x N
 * identity, no (E,H,Np,N) Y state.  `A` is a contiguous (E,H,N,N) fp32 device
 * array.  Of *p the fields v, out, Dv, dtype_v, v_stride and out_stride are not
 * read; size the workspace for Dv = D and dtype_v = dtype_qk.  Variants AUTO,
 * GENERIC and STAGED (they select the kernels of the T steps);
 * MA_ERR_UNSUPPORTED for the one-launch variants and for padded sequences
 * beyond what one workgroup's LDS holds (M*B + 64*M floats <= 160 KB). */
int ma_matrix(const ma_fwd_params* p, float* A, void* stream);

/* Backward pass.  The reference has no backward code: it differentiates
 * monarch_attention_torch (ma/ma_torch.py:65-108) with PyTorch autograd, which
 * is what training through the operator uses (experiments/gps/train.py:34).
 * ma_bwd is that derivative: given the inputs of a forward call and the
 * gradient of its output it writes the gradients of q, k and v.  The forward
 * state is not kept between the two calls: ma_bwd runs the T steps again
 * (kernels chosen by fwd.variant: AUTO, GENERIC or STAGED), keeping every
 * step's state in its workspace, then walks the steps backwards in fp32.
 *   fwd            the forward call's arguments; fwd.out is not read;
 *                  fwd.workspace / workspace_bytes: >= ma_bwd_workspace_bytes()
 *   dout           (E,H,N,Dv) dtype_v, element strides dout_stride
 *   dq, dk / dv    (E,H,N,D) dtype_qk / (E,H,N,Dv) dtype_v, written in full
 * MA_ERR_UNSUPPORTED for the one-launch variants and for M > 6144 or B > 4096. */
typedef struct ma_bwd_params {
    ma_fwd_params fwd;
    const void* dout;
    void* dq;
    void* dk;
    void* dv;
    int64_t dout_stride[3];
    int64_t dq_stride[3];
    int64_t dk_stride[3];
    int64_t dv_stride[3];
} ma_bwd_params;

uint64_t ma_bwd_workspace_bytes(const ma_bwd_params* p);
int ma_bwd(const ma_bwd_params* p, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MA_HIP_H_ */
