/* libhdla_hip.so -- C ABI of the MI355X (gfx950) kernels for HDLA's rank-2 DPLR delta-rule linear attention.
 *
 * This is the boundary a host binding talks to (ctypes in this repository; any FFI works): plain pointers
 * and sizes, no C++ or torch types.  It stands in for the reference's Python launcher layer, which is the
 * level at which its Triton kernels are driven:
 *
 *   hdla_chunk_fwd      <-  chunk_hrdplr_fwd                     HRDPLR/hrdplr.py:25-99
 *                           (chunk_fwd_intra_dplr_fn HRDPLR/fwd_func.py:16, fwd_prepare_wy_repr :153,
 *                            chunk_dplr_fwd_h :210, chunk_dplr_fwd_o :274 and fla's chunk_rwkv6_fwd_cumsum)
 *   hdla_chunk_bwd      <-  ChunkDPLRDeltaRuleFunction.backward   HRDPLR/hrdplr.py:149-284
 *                           (chunk_dplr_bwd_dAu HRDPLR/bwd_func.py:18, _dhu :63, _dv :125, _bwd_o :155,
 *                            _bwd_wy :218, _bwd_dqk_intra :274)
 *   hdla_recurrent_fwd  <-  fused_recurrent_dplr_delta_rule_fwd   HRDPLR/recurrent.py:121-177
 *   hdla_param_*        <-  the same three with parameterize_a_b (HRDPLR/hdla_custom.py:19-43) folded in
 *
 * and, for the layer around the operator (HRDPLR/hdla_custom.py:45-350):
 *
 *   hdla_normalize_*    <-  NormalizeTriton   HRDPLR/normalizations/normalize/normalize/normalize_triton.py:255-449
 *   hdla_layer_pre_*, hdla_logsigmoid_*   <-  the elementwise steps between projections and operator
 *                                             HRDPLR/hdla_custom.py:214-251
 *   hdla_skinny_wgrad   <-  the weight gradient of the low-rank up-projections (a BLAS call inside autograd)
 *
 * Conventions
 *   - All tensor pointers are DEVICE pointers to contiguous, 16-byte aligned buffers owned by the caller.
 *     Layouts are the reference's (head_first = False): q,k,gk [B,T,H,K]; v,o,do [B,T,H,V];
 *     a,b [B,T*R,H,K] with row t*R + r (HRDPLR/recurrent.py:66-67); states [N,H,K,V] fp32.
 *   - The library allocates nothing.  The caller passes a workspace of hdla_workspace_bytes() bytes
 *     (256-byte aligned); its contents are scratch and may be discarded after the call.
 *   - Calls are asynchronous on `stream` (a hipStream_t passed as void*; NULL = the default stream), never
 *     synchronise, keep no global mutable state and are reentrant as long as workspaces are distinct.
 *   - Return value: 0 = success, < 0 = argument error detected on the host before any launch (see
 *     hdla_strerror), > 0 = a hipError_t from a kernel launch.
 *   - Supported: R = 2; K, V in {64, 128} (the token-serial entry points also 256); in_dtype bf16 or fp32; gk fp32,
 *     or bf16 when in_dtype is bf16.
 *     gk (log-space decay, <= 0) may be arbitrarily strong: where a channel loses more than e^-70 within eight
 *     tokens the chunk's scores are formed by passes whose exponents cannot overflow, as the reference's
 *     re-centred sub-chunks are (HRDPLR/fwd_triton.py:420-463).
 */
#ifndef HDLA_HIP_H
#define HDLA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HDLA_VERSION 200

enum { HDLA_BF16 = 0, HDLA_FP32 = 1 };

enum {
    HDLA_OK = 0,
    HDLA_ERR_NULL = -1,        /* a required pointer is NULL */
    HDLA_ERR_SHAPE = -2,       /* unsupported K/V, non-positive dimension, or grid limit exceeded */
    HDLA_ERR_RANK = -3,        /* R != 2 */
    HDLA_ERR_DTYPE = -4,       /* unknown dtype code or unsupported combination */
    HDLA_ERR_WORKSPACE = -5,   /* workspace NULL, misaligned or too small */
    HDLA_ERR_ALIGN = -6,       /* a tensor pointer is not 16-byte aligned */
    HDLA_ERR_SEQ = -7,         /* cu_seqlens given with B != 1, or N inconsistent with B */
    HDLA_ERR_STATIC_LIMIT = -8,/* hdla_chunk_fwd_static: the shape needs more than HDLA_STATIC_WORKSPACE_BYTES */
    HDLA_ERR_ROUTE = -9        /* unknown route, negative segments, or HDLA_ROUTE_FUSED on a shape it is not built for */
};

/* Launch plans of the chunked entry points.  HDLA_ROUTE_CLASSIC: one kernel prepares every chunk (scores,
 * (I - A_ab)^-1, w, u, gated copies) into the workspace and the state scans read it back, a head's value columns
 * split over workgroups.  HDLA_ROUTE_FUSED (bf16 inputs, K = V = 64): the preparation runs inside the scan kernels'
 * workgroups and reaches the scan through LDS; a sequence is cut into `segments` time segments whose affine maps are
 * chained afterwards, so that few (sequence, head) pairs still fill the device.  HDLA_ROUTE_AUTO takes the fused route
 * where it is built.  Both routes compute the same function; they differ in rounding only where segments > 1. */
enum { HDLA_ROUTE_AUTO = 0, HDLA_ROUTE_CLASSIC = 1, HDLA_ROUTE_FUSED = 2 };
#define HDLA_FUSED_ABORTED 0x48444c00

typedef struct hdla_dims {
    int32_t B, T, H, K, V, R;
    int32_t N;                 /* sequences: B without cu_seqlens, else len(cu_seqlens) - 1 (and B == 1) */
    int32_t in_dtype;          /* q,k,v,a,b,o,do and dq,dk,dv,da,db */
    int32_t gk_dtype;          /* gk and dgk */
    float scale;               /* applied to q (HRDPLR/hrdplr.py:302) */
    const int64_t* cu_seqlens; /* DEVICE int64[N+1] cumulative sequence starts on the T axis, or NULL */
    int32_t route;             /* HDLA_ROUTE_*; 0 = the library chooses */
    int32_t segments;          /* fused route: time segments per sequence (at most 64); 0 = the library chooses */
} hdla_dims;

/* Byte offsets of the named intermediates inside the workspace (0 = not part of this pass); for tests and
 * debugging: after hdla_chunk_bwd every stage's output is still there.  "tiles" are 16x16 blocks in MFMA
 * fragment order (element 4*lane + i of a block is row lane%16, inner index 4*(lane/16) + i; consecutive
 * tile pairs are stored interleaved, element 8*lane + 4*which + i), "rows" are row-major, all laid out
 * [H][nch][...].  W, BGT, KGT, QG, AQB, AQK, EGL are parts of one block per (head, chunk) slot: the value given
 * is the offset for slot 0 and consecutive slots are SA_STRIDE bytes apart; likewise QGT, AQBT
 * with SB_STRIDE.  On the fused route the scans' operands never reach the workspace: only TM, HC, DHC, DVN, STRONG
 * (and W, UT where chunk_grad reads them instead of rebuilding them: the hdla_param_ forms, fp32 decays beside bf16
 * inputs) are written, in the backward pass. */
typedef struct hdla_ws_layout {
    int64_t nch;               /* chunk slots per head */
    int64_t W, UT, KGT, BGT, VTT, EGL, QG, AQK, AQB, AQBT, QGT, TM, HC, DHC, DVN;
    int64_t STRONG;            /* int32 per (head, chunk) slot: nonzero where the chunk takes the strong-decay route */
    int64_t SA_STRIDE, SB_STRIDE;
    int64_t CHUNK_OFF, CHUNK_SEQ;  /* with cu_seqlens: int32[N+1] first chunk slot of each sequence, followed by int32[N]
                                    * the sequences in the order the scans start them (most chunks first); int32[nch] the
                                    * sequence of each chunk slot */
    int64_t total;
    int64_t ERR;               /* fused route: int32 that reads (HDLA_FUSED_ABORTED | 1..3) only if a wave's bounded wait for
                                * another wave ran out (the kernels then stop early and the results are invalid); the
                                * library never clears it; -1 on the classic route */
} hdla_ws_layout;

int hdla_version(void);
const char* hdla_strerror(int code);

/* Workspaces by pass.  HDLA_PASS_FWD and HDLA_PASS_BWD are the scratch of hdla_chunk_fwd / hdla_chunk_bwd (contents
 * disposable after the call).  HDLA_PASS_FWD_KEEP is the buffer hdla_chunk_fwd_keep fills and hdla_chunk_bwd_kept
 * reads (it must survive from the one to the other), HDLA_PASS_BWD_KEPT the scratch of hdla_chunk_bwd_kept.
 * hdla_workspace_bytes returns 0 for invalid dims or pass. */
enum { HDLA_PASS_FWD = 0, HDLA_PASS_BWD = 1, HDLA_PASS_FWD_KEEP = 2, HDLA_PASS_BWD_KEPT = 3 };
size_t hdla_workspace_bytes(const hdla_dims* dims, int pass);
int hdla_workspace_layout(const hdla_dims* dims, int pass, hdla_ws_layout* out);

/* Chunked forward (HRDPLR/hrdplr.py:25-99).  h0 and ht are optional (NULL): zero initial state / final state
 * not wanted.  o has q's dtype (HRDPLR/hrdplr.py:144), ht is fp32 (HRDPLR/fwd_func.py:244). */
int hdla_chunk_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                   const void* b, const void* gk, const float* h0, void* o, float* ht,
                   void* workspace, size_t workspace_bytes, void* stream);

/* hdla_chunk_fwd for callers that cannot allocate device memory and have no workspace to pass: code under HIP graph
 * capture, tight serving loops (a prefill or a burst of a few tokens per sequence), harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  Same arguments and results as hdla_chunk_fwd without the
 * workspace: the kernels use an array of HDLA_STATIC_WORKSPACE_BYTES bytes that is part of the library's device
 * code (every GPU the library runs on holds it until the process ends); the call allocates and frees nothing.
 * A shape whose hdla_workspace_bytes(dims, 0) exceeds that size is refused with HDLA_ERR_STATIC_LIMIT (K = V = 64,
 * bf16: up to 3276 (16-token chunk, head) pairs, e.g. one sequence of 3276 tokens with 16 heads).  All calls on
 * one GPU share the array: calls that may overlap on one GPU (different streams, different threads) race; calls
 * on one stream are safe.  The array's device address is looked up on the first call on each device; make that
 * call outside graph capture. */
#define HDLA_STATIC_WORKSPACE_BYTES (64u << 20)
int hdla_chunk_fwd_static(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                          const void* b, const void* gk, const float* h0, void* o, float* ht, void* stream);

/* Chunked backward (HRDPLR/hrdplr.py:149-284): recomputes the forward intermediates from the inputs, then
 * writes dq,dk,dv,da,db (in_dtype), dgk (gk_dtype) and, if dh0 != NULL, dh0 (fp32).  dht may be NULL. */
int hdla_chunk_bwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                   const void* b, const void* gk, const float* h0, const void* d_o, const float* dht,
                   void* dq, void* dk, void* dv, void* da, void* db, void* dgk, float* dh0,
                   void* workspace, size_t workspace_bytes, void* stream);

/* hdla_chunk_fwd / hdla_chunk_bwd (or, with beta given, hdla_param_chunk_fwd / _bwd: a, b, da, db are then ignored and
 * may be NULL) with the states at the segment boundaries handed from the forward to the backward pass.  On the fused
 * route with several segments the backward pass needs the state entering every segment before it can checkpoint the
 * states inside it.  The forward pass has them: given `boundary` (hdla_boundary_bytes(dims) bytes, 16-byte aligned;
 * 64 KiB per (sequence, head, segment) at K = V = 64, i.e. under 2 % of the inputs of 512-token segments) it leaves them
 * there, and the backward pass reads them instead of re-deriving them from the inputs with one more pass over them
 * (which is what hdla_chunk_bwd does, and hdla_chunk_bwd_b with boundary = NULL).  The reference keeps the inputs only
 * (ctx.save_for_backward, HRDPLR/hrdplr.py:137) and recomputes everything (:161-198); the record is what this route
 * adds to that.  hdla_boundary_bytes returns 0 where the route has no such record (classic route, one segment):
 * boundary is then ignored. */
size_t hdla_boundary_bytes(const hdla_dims* dims);
int hdla_chunk_fwd_b(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a, const void* b,
                     const void* beta, const void* gk, const float* h0, void* o, float* ht, void* boundary,
                     size_t boundary_bytes, void* workspace, size_t workspace_bytes, void* stream);
int hdla_chunk_bwd_b(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a, const void* b,
                     const void* beta, const void* gk, const float* h0, const void* d_o, const float* dht, void* dq,
                     void* dk, void* dv, void* da, void* db, void* dbeta, void* dgk, float* dh0, const void* boundary,
                     size_t boundary_bytes, void* workspace, size_t workspace_bytes, void* stream);

/* The same operator with a and b formed inside the kernels the way the HDLA layer forms them
 * (parameterize_a_b, HRDPLR/hdla_custom.py:19-43, called at :290 right before the operator):
 *     f = exp(gk),  s = sum_c k_c^2 f_c,   a_1 = -beta k,  a_2 = beta k (beta s - f),   b_1 = f k,  b_2 = k
 * (identical to the reference's a_2 = a_t2 + a_t1 sum(b_t1 a_t2); the decay is (I - beta k k^T) Diag(f) (I - beta k k^T)),
 * with a and b rounded to the input dtype as the layer's .to(dtype) does (:301-304).  beta is [B,T,H] in the input
 * dtype.  a and b are never materialised: neither read here nor written by a caller.  The backward pass returns
 * dbeta [B,T,H] and folds the gradients of a and b into dk and dgk. */
int hdla_param_chunk_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* beta,
                         const void* gk, const float* h0, void* o, float* ht,
                         void* workspace, size_t workspace_bytes, void* stream);
int hdla_param_chunk_bwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* beta,
                         const void* gk, const float* h0, const void* d_o, const float* dht,
                         void* dq, void* dk, void* dv, void* dbeta, void* dgk, float* dh0,
                         void* workspace, size_t workspace_bytes, void* stream);

/* The pair for callers that would rather spend memory than time: hdla_chunk_fwd_keep is hdla_chunk_fwd (or, with beta
 * given, hdla_param_chunk_fwd: a and b are then ignored and may be NULL) whose per-chunk intermediates -- the operands
 * of the state scans, (I - A_ab)^-1, the strong-decay flags -- are written into a buffer `kept` of
 * hdla_workspace_bytes(dims, HDLA_PASS_FWD_KEEP) bytes that the caller holds until the backward pass;
 * hdla_chunk_bwd_kept is hdla_chunk_bwd (hdla_param_chunk_bwd with beta: dbeta is written, da and db are not) that reads
 * them there instead of recomputing them from the inputs, which saves the backward pass its first kernel.  The reference
 * keeps only the inputs between the passes and recomputes (ctx.save_for_backward at HRDPLR/hrdplr.py:137, recompute at
 * :161-198); these two trade that for about 1.6x the inputs' bytes of extra memory held between the passes.  `kept` is
 * only read by the backward call (it can be used again); `workspace` is scratch of
 * hdla_workspace_bytes(dims, HDLA_PASS_BWD_KEPT) bytes.  Same dims, inputs and stream ordering as the forward call. */
int hdla_chunk_fwd_keep(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                        const void* b, const void* beta, const void* gk, const float* h0, void* o, float* ht,
                        void* kept, size_t kept_bytes, void* stream);
int hdla_chunk_bwd_kept(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                        const void* b, const void* beta, const void* gk, const float* h0, const void* d_o,
                        const float* dht, void* dq, void* dk, void* dv, void* da, void* db, void* dbeta, void* dgk,
                        float* dh0, void* kept, size_t kept_bytes, void* workspace, size_t workspace_bytes,
                        void* stream);

/* Profiling / debugging aid with no counterpart in the reference: runs only the kernels selected by `stages`
 * (a bit mask) of the forward (pass 0) or backward (pass 1) launch sequence, in order, on the same workspace, so
 * that a caller can bracket each kernel with events on `stream`.  A stage reads what the earlier stages left
 * in the workspace.  Unused tensor arguments of the other pass may be NULL. */
enum {
    HDLA_STAGE_PREP = 1,        /* chunk table (with cu_seqlens) + prep kernel (fused route: the table only) */
    HDLA_STAGE_SCAN_FWD = 2,    /* forward state scan (writes o in pass 0; state checkpoints in pass 1); on the fused route
                                 * the kernel that prepares and scans (forward kernel in pass 0, checkpoint kernel in pass 1) */
    HDLA_STAGE_SCAN_BWD = 4,    /* reverse state-gradient scan (pass 1 only) */
    HDLA_STAGE_CHUNK_GRAD = 8,  /* per-chunk gradient assembly (pass 1 only) */
    HDLA_STAGE_CHAIN = 16,      /* fused route with several segments only.  Pass 0: the kernel that chains the segments and
                                 * completes the outputs.  Pass 1: what a backward pass without a boundary record runs first
                                 * (summary kernel + chaining); it leaves the states entering the segments in the workspace,
                                 * where later calls without this stage find them */
    HDLA_STAGE_ALL = 31
};
int hdla_chunk_stages(const hdla_dims* dims, int pass, int stages, const void* q, const void* k, const void* v,
                      const void* a, const void* b, const void* gk, const float* h0, void* o, float* ht,
                      const void* d_o, const float* dht, void* dq, void* dk, void* dv, void* da, void* db, void* dgk,
                      float* dh0, void* workspace, size_t workspace_bytes, void* stream);

/* Token-serial recurrence over T tokens per sequence (HRDPLR/recurrent.py:121-177), forward only.
 * reverse != 0 walks each sequence from its last token to its first (recurrent.py:63,108). */
int hdla_recurrent_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                       const void* b, const void* gk, int reverse, const float* h0, void* o, float* ht,
                       void* stream);

/* The same recurrence with the rank terms of the HDLA layer formed per token inside the kernel from
 * (beta [B,T,H], k, gk = log f) instead of read from a and b: parameterize_a_b, HRDPLR/hdla_custom.py:19-43,
 * followed by fused_recurrent_dplr_delta_rule_fwd, HRDPLR/recurrent.py:121-177.  beta has the input dtype and
 * must not be NULL (also when T = 0: it selects the mode). */
int hdla_param_recurrent_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* beta,
                             const void* gk, int reverse, const float* h0, void* o, float* ht, void* stream);

/* Fused normalisation with an optional sigmoid gate, the operator the HDLA layer applies around the attention
 * operator: _normalize_fwd / _normalize_bwd, HRDPLR/normalizations/normalize/normalize/normalize_triton.py:21-253
 * (NormalizeTriton.forward :256-352, .backward :354-449) for use_mean = False, no bias, no residual.
 * A tensor is `rows` rows of G groups of E channels, contiguous; per group
 *     x' = x * sigmoid(gate) (gate_pos 1),  sigma = sqrt(sum x'^2 / E + eps),
 *     o = (c / sqrt(E)) * x' / sigma * weight  [* sigmoid(gate), gate_pos 2].
 * rms norm over a row: G = 1, c = sqrt(E) (normalizations/utils.py:35-39); group rms norm: c = sqrt(E), G groups
 * (:47-50); l2_norm: G = 1, c = 1, no weight (normalizations/l2_norm.py:4-14).
 * E must be a multiple of 16 bytes' worth of elements and at most 16384 (bf16) / 8192 (fp32). */
typedef struct hdla_norm_dims {
    int64_t rows;              /* product of the leading dimensions */
    int32_t G, E;              /* groups per row, channels per group */
    int32_t dtype;             /* x, gate, o, do, dx, dgate */
    int32_t weight_dtype;      /* weight [G*E] (ignored when weight is NULL) */
    int32_t gate_pos;          /* 0 = no gate, 1 = before the norm ("pre"), 2 = after it ("post") */
    float c, eps;
} hdla_norm_dims;

/* weight and gate may be NULL (gate only with gate_pos 0). */
int hdla_normalize_fwd(const hdla_norm_dims* dims, const void* x, const void* weight, const void* gate, void* o,
                       void* stream);
/* Backward pass; sigma is recomputed.  dw: fp32 [G*E], required iff weight is given; it is summed over rows in a
 * fixed order through `workspace` (hdla_normalize_workspace_bytes() bytes, 16-byte aligned; not needed without a
 * weight).  dgate is required iff gate_pos != 0. */
int hdla_normalize_bwd(const hdla_norm_dims* dims, const void* x, const void* weight, const void* gate,
                       const void* d_o, void* dx, void* dgate, float* dw, void* workspace, size_t workspace_bytes,
                       void* stream);
size_t hdla_normalize_workspace_bytes(const hdla_norm_dims* dims);

/* What the HDLA layer does between its projections and the operator, one pass per direction
 * (HRDPLR/hdla_custom.py:214-251): q = silu(q_raw), k = silu(k_raw), v = silu(v_raw), each l2-normalised per head when
 * its flag is set (x / sqrt(sum x^2 + D eps), HRDPLR/normalizations/l2_norm.py:4-14; the layer always sets norm_k), and
 * beta = beta_scale * sigmoid(bet_raw).  The raw inputs are column ranges of one row-major matrix y [rows, ldy]
 * (a projection output): q_raw of head h at columns col_q + h*D .. + D, likewise k, v; bet_raw at col_beta + h
 * (col_beta < 0: no beta).  Outputs are contiguous [rows, H, D] (q, k, v) and [rows, H] (beta).
 * D * element size must be 16 bytes times a power of two <= 64; ldy and the q/k/v column offsets multiples of 16 bytes. */
typedef struct hdla_pre_dims {
    int64_t rows;
    int32_t H, D;
    int32_t dtype;
    int32_t ldy, col_q, col_k, col_v, col_beta;
    int32_t norm_q, norm_k, norm_v;
    float beta_scale, eps;
} hdla_pre_dims;
int hdla_layer_pre_fwd(const hdla_pre_dims* dims, const void* y, void* q, void* k, void* v, void* beta, void* stream);
/* Backward pass: from y and the gradients of the four outputs, the gradient of y's four column ranges, written in
 * place into dy [rows, ldy]; the other columns of dy are not touched. */
int hdla_layer_pre_bwd(const hdla_pre_dims* dims, const void* y, const void* dq, const void* dk, const void* dv,
                       const void* dbeta, void* dy, void* stream);
/* log_f = logsigmoid(f) (HRDPLR/hdla_custom.py:219) and its gradient df = dlog_f * sigmoid(-f), elementwise over n
 * contiguous elements (n a multiple of 16 bytes' worth). */
int hdla_logsigmoid_fwd(int dtype, int64_t n, const void* x, void* y, void* stream);
int hdla_logsigmoid_bwd(int dtype, int64_t n, const void* x, const void* dy, void* dx, void* stream);

/* dW [K, N] = dY [M, K]^T * X0 [M, N], bf16 with fp32 accumulation, for N = 64 or 128 and K a multiple of 64: the
 * weight gradient of the layer's Linear(head_dim -> embed_dim) projections (second halves of f_proj and output_gate,
 * HRDPLR/hdla_custom.py:117-121,151-155; in the reference a BLAS call inside autograd) with dY [M, embed_dim] the
 * gradient of their output and X0 [M, head_dim] their input.  ldy, ldx: row strides in elements (multiples of 8);
 * dW is contiguous [K, N] (the weight's layout).  The rows are split over workgroups; partial results go through
 * `workspace` (hdla_skinny_wgrad_workspace_bytes() bytes, 16-byte aligned) and are added in a fixed order. */
int hdla_skinny_wgrad(int dtype, int64_t M, int32_t N, int32_t K, const void* dY, int64_t ldy, const void* X0,
                      int64_t ldx, void* dW, void* workspace, size_t workspace_bytes, void* stream);
size_t hdla_skinny_wgrad_workspace_bytes(int dtype, int64_t M, int32_t N, int32_t K);

/* Measurement aid; it has no counterpart in the reference.  One launch of a kernel that reads `n_read` (0..3)
 * buffers and writes `n_write` (0..2) buffers of `bytes` bytes each (a multiple of 16; every pointer 16-byte
 * aligned) and does nothing else.  Supported mixes (reads:writes): 1:0, 0:1, 1:1, 2:1, 3:1, 1:2; others return
 * HDLA_ERR_SHAPE.  Its traffic is known exactly, which is what hardware traffic counters are scaled by, and the
 * rate it reaches is the rate HBM sustains for that mix. */
int hdla_calib_stream(const void* const* reads, int n_read, void* const* writes, int n_write, size_t bytes,
                      void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HDLA_HIP_H */
