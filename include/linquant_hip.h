/* C ABI of liblinquant_hip.so: MI355X (gfx950) INT8 chunkwise linear-recurrence prefill.
 *
 * Every entry point takes a pointer to a plain args struct (device pointers, sizes, element
 * strides, scalars, flags) and the HIP stream to launch on, and returns 0 or a negative code:
 *   LQ_E_NULL  (-14) a required pointer is missing
 *   LQ_E_SHAPE (-22) unsupported size / stride / alignment / flag
 *   LQ_E_LAUNCH (-5) hipGetLastError() reported a launch failure
 *   LQ_E_STATE (-11) the call needs set-up that cannot run now (stream under graph capture)
 * Entry points never allocate, never synchronise, never throw and keep no mutable global state:
 * the caller owns every buffer (inputs, outputs, intermediates) and may call concurrently on
 * different streams.  All strides are in elements of the tensor's dtype.  "device float*" scalars
 * (dt_scale, A_log_scale, D_scale) are 0-dim device tensors read inside the kernel, as in the
 * reference, so no host synchronisation is needed to obtain them.
 *
 * Each declaration cites the reference (ntumm120/LinQuant) interface it replaces.
 */
#ifndef LINQUANT_HIP_H
#define LINQUANT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef __HIP__
#ifndef HIP_INCLUDE_HIP_HIP_RUNTIME_API_H
typedef struct ihipStream_t* hipStream_t;
#endif
#endif

#define LQ_E_NULL (-14)
#define LQ_E_SHAPE (-22)
#define LQ_E_LAUNCH (-5)
#define LQ_E_STATE (-11)

/* element types accepted for the raw dt input */
#define LQ_DT_F16 0
#define LQ_DT_F32 1
#define LQ_DT_I8 2
#define LQ_DT_BF16 3

/* ABI version; bumped whenever a struct layout changes. */
int lq_abi_version(void);
/* sizeof() of the named args struct as compiled into the library (negative if unknown); lets a binding
 * check its own struct layout before the first call. */
int lq_args_size(const char* name);

/* ------------------------------------------------------------------------------------------
 * Mamba-2 SSD pipeline (SSDi8 lineage).  Layouts: x (B,L,H,P) fp16 with arbitrary batch/seq/head
 * strides and unit P stride (a view of xBC); B/C (B,L,G,N); dt, dA_cumsum (B,H,nc,Q) fp32
 * contiguous; chunk states (B,nc,H,P,N) int8 contiguous.
 * ------------------------------------------------------------------------------------------ */

/* replaces _quant_chunk_cumsum_fwd, linquant/kernels/mamba2/chunk_cumsum.py:77-100 (kernel :27-74) */
typedef struct {
  const void* dt;            /* (B,L,H) raw dt, dtype dt_dtype, strides below */
  int32_t dt_dtype;          /* LQ_DT_* */
  int64_t dt_stride_b, dt_stride_l, dt_stride_h;
  const float* dt_scale;     /* device scalar */
  const int8_t* A_log;       /* (H,) int8 */
  int64_t A_log_stride_h;
  const float* A_log_scale;  /* device scalar */
  const float* dt_bias;      /* (H,) fp32 or NULL */
  int64_t dt_bias_stride_h;
  float* dt_out;             /* (B,H,nc,Q) fp32 contiguous */
  float* dA_cumsum;          /* (B,H,nc,Q) fp32 contiguous */
  int32_t batch, seqlen, nheads, chunk_size;
  int32_t dt_softplus;
  float dt_min, dt_max;
} lq_chunk_cumsum_args;
int lq_chunk_cumsum(const lq_chunk_cumsum_args* args, hipStream_t stream);

/* replaces _quant_chunk_state_fwd_xfp_static_int8, linquant/kernels/mamba2/chunk_state.py:258-349
 * (kernel :72-255): value-side absorption, x quantized per tile with alpha_hp against INT8 B. */
typedef struct {
  const void* x;             /* (B,L,H,P) fp16, unit P stride */
  int64_t x_stride_b, x_stride_l, x_stride_h;
  const int8_t* B;           /* (B,L,G,N) int8, unit N stride */
  int64_t B_stride_b, B_stride_l, B_stride_g;
  const float* dt;           /* (B,H,nc,Q) fp32 contiguous */
  const float* dA_cumsum;    /* (B,H,nc,Q) fp32 contiguous */
  const float* alpha_hp;     /* (H,P) view; stride_p == 0 means one scalar per head */
  int64_t alpha_stride_h, alpha_stride_p;
  const float* bscale_g;     /* (G,) */
  int64_t bscale_stride_g;
  const float* out_qscale;   /* (H,P) view, stride_p may be 0 */
  int64_t oqs_stride_h, oqs_stride_p;
  int8_t* states;            /* (B,nc,H,P,N) int8, contiguous but for the batch stride */
  int32_t batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size;
  int64_t states_stride_b;   /* elements between batch rows of `states`; 0 = dense (nc*H*P*N) */
} lq_chunk_state_value_args;
int lq_chunk_state_value(const lq_chunk_state_value_args* args, hipStream_t stream);

/* replaces _chunk_state_keyside_fwd, linquant/kernels/mamba2/chunk_state_keyside.py:342-424
 * (kernel :163-330): key-side absorption, x quantized with x_scale_hp, fp16 B weighted by the gate
 * and quantized in-loop with the raw-amax b_gate_scale (codes = rint(gate*B*127/b_gate)). */
typedef struct {
  const void* x;             /* (B,L,H,P) fp16, unit P stride */
  int64_t x_stride_b, x_stride_l, x_stride_h;
  const void* B;             /* (B,L,G,N) fp16, unit N stride */
  int64_t B_stride_b, B_stride_l, B_stride_g;
  const float* dt;
  const float* dA_cumsum;
  const float* x_scale_hp;   /* (H,P) view */
  int64_t xs_stride_h, xs_stride_p;
  const float* out_qscale;   /* (H,P) view */
  int64_t oqs_stride_h, oqs_stride_p;
  const float* b_gate_scale; /* 4-D broadcastable (B,nc,H,N); size-1 dims carry stride 0 */
  int64_t bgs_stride_b, bgs_stride_c, bgs_stride_h, bgs_stride_n;
  int8_t* states;            /* (B,nc,H,P,N) int8, contiguous but for the batch stride */
  int32_t batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size;
  int64_t states_stride_b;   /* elements between batch rows of `states`; 0 = dense (nc*H*P*N) */
  float* b_rowmax;           /* NULL, or (B,L,G) fp32 scratch: the call first fills it with max_n |B[b,l,g,n]| and then leaves
                                out every 64-token slab whose gated key codes are provably all zero (same result, bit for
                                bit; see the kernel's header).  Contents undefined on entry. */
  int32_t b_rowmax_ready;    /* 1: b_rowmax already holds the row maxima (lq_split_rotate_quant_xBC wrote them beside b_fp):
                                the pre-pass over B is left out */
} lq_chunk_state_key_args;
int lq_chunk_state_key(const lq_chunk_state_key_args* args, hipStream_t stream);

/* replaces _fixedpoint_state_passing_fwd, linquant/kernels/mamba2/state_passing.py:96-121
 * (kernel :25-93). out[:,0] = 0, out[:,c+1] = state after chunk c, final = state after the last. */
typedef struct {
  const int8_t* states;      /* (B,nc,H,dim) int8 */
  int64_t states_stride_b, states_stride_c, states_stride_h, states_stride_d;
  const float* dA_chunk_cumsum; /* (B,H,nc) view: last cumsum entry of every chunk */
  int64_t dA_stride_b, dA_stride_h, dA_stride_c;
  int8_t* out;               /* (B,nc,H,dim) int8 */
  int64_t out_stride_b, out_stride_c, out_stride_h, out_stride_d;
  int8_t* final_states;      /* (B,H,dim) int8 or NULL */
  int64_t final_stride_b, final_stride_h, final_stride_d;
  int32_t batch, nchunks, nheads, dim;
  int32_t gate_shift;        /* fractional bits of the fixed-point gate, 0..15 (reference: 7) */
  int32_t vec_hint;          /* 0 = auto; 4/8/16 = bytes per thread to try first */
  int32_t in_place;          /* 0: `states` and `out` are distinct buffers.  1: they are one buffer of nc + 1 chunk slots per
                                batch row, out = slot 0, states = slot 1 (same strides): slot c + 1 holds the local state of
                                chunk c on entry and the state entering chunk c + 1 on return, slot 0 is zero-filled.  A
                                (batch, head) all of whose gates quantize to zero then needs no pass at all: the state
                                entering chunk c + 1 is the local state of chunk c, which is already in place. */
} lq_state_passing_args;
int lq_state_passing(const lq_state_passing_args* args, hipStream_t stream);

/* replaces _quant_bmm_chunk_fwd, linquant/kernels/mamba2/bmm_chunk.py:142-217 (kernel :49-139):
 * CB_i8 = clamp(rint(C_i8 . B_i8^T * (sC*sB/S_cb)), +-127) per (batch, chunk, group). */
typedef struct {
  const int8_t* a;           /* C: (B,L,G,N) int8, unit N stride */
  int64_t a_stride_b, a_stride_l, a_stride_g;
  const void* b;             /* B: (B,L,G,N) int8, or fp16 when b_is_fp */
  int64_t b_stride_b, b_stride_l, b_stride_g;
  const float* a_scale;      /* (G,) */
  const float* b_scale;      /* (G,) */
  const float* cb_scale;     /* (G,) static output scale */
  int8_t* out;               /* (B,nc,G,Q,Q) int8 contiguous */
  int32_t batch, seqlen, ngroups, dstate, chunk_size;
  int32_t b_is_fp;
} lq_bmm_chunk_args;
int lq_bmm_chunk(const lq_bmm_chunk_args* args, hipStream_t stream);

/* replaces _quant_chunk_scan_fwd, linquant/kernels/mamba2/chunk_scan_v2.py:259-366 (kernel :56-256). */
typedef struct {
  const int8_t* cb;          /* (B,nc,G,Q,Q) int8 contiguous */
  const void* x;             /* (B,L,H,P) fp16, unit P stride */
  int64_t x_stride_b, x_stride_l, x_stride_h;
  const float* dt;           /* (B,H,nc,Q) */
  const float* dA_cumsum;    /* (B,H,nc,Q) */
  const int8_t* C;           /* (B,L,G,N) int8, unit N stride */
  int64_t C_stride_b, C_stride_l, C_stride_g;
  const float* C_scale;      /* (G,) */
  const int8_t* states;      /* (B,nc,H,P,N) int8 contiguous: state entering each chunk */
  const float* states_scale; /* (H,P) view, stride_p may be 0 */
  int64_t ss_stride_h, ss_stride_p;
  const int8_t* D;           /* (H,) or (H,P) int8, or NULL */
  int64_t D_stride_h;
  int32_t D_has_hdim;
  const float* D_scale;      /* device scalar (ignored when D is NULL) */
  const float* cb_scale;     /* (G,) */
  void* out;                 /* (B,L,H,P) fp16 contiguous */
  int32_t batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size;
  int64_t states_stride_b;   /* elements between batch rows of `states`; 0 = dense (nc*H*P*N) */
  int32_t heads_hint;        /* heads of one group that a workgroup walks one after the other (they share the C rows and CB
                                codes it keeps in registers, and each head's loads overlap the previous head's arithmetic);
                                0 = chosen from the grid size; clamped to heads per group.  Same bits for every value. */
} lq_chunk_scan_args;
int lq_chunk_scan(const lq_chunk_scan_args* args, hipStream_t stream);

/* replaces _quant_mamba_chunk_scan_combined_fwd, linquant/kernels/mamba2/ssd_combined.py:19-131, as one call: the five
 * stages above launched back to back on `stream` (cumsum -> chunk state -> state passing -> C.B^T -> chunk scan), with
 * the intermediates the reference allocates per call (dt, dA_cumsum, chunk states, passed states, CB) laid out in one
 * caller-supplied workspace.  Field meanings as in the per-stage structs; keyside selects lq_chunk_state_key (x_scale_hp,
 * b_fp, b_gate_scale) or lq_chunk_state_value (qB, alpha_hp, bscale_g), and the B operand of C.B^T with it. */
typedef struct {
  const void* x;             /* (B,L,H,P) fp16, unit P stride */
  int64_t x_stride_b, x_stride_l, x_stride_h;
  const void* dt;            /* (B,L,H) raw dt */
  int32_t dt_dtype;
  int64_t dt_stride_b, dt_stride_l, dt_stride_h;
  const float* dt_scale;     /* device scalar */
  const int8_t* A_log;       /* (H,) */
  int64_t A_log_stride_h;
  const float* A_log_scale;  /* device scalar */
  const float* dt_bias;      /* (H,) or NULL */
  int64_t dt_bias_stride_h;
  int32_t dt_softplus;
  float dt_min, dt_max;
  const int8_t* qB;          /* (B,L,G,N) int8 (value side), unit N stride */
  int64_t qB_stride_b, qB_stride_l, qB_stride_g;
  const void* b_fp;          /* (B,L,G,N) fp16 (key side), unit N stride */
  int64_t bfp_stride_b, bfp_stride_l, bfp_stride_g;
  const int8_t* qC;          /* (B,L,G,N) int8, unit N stride */
  int64_t qC_stride_b, qC_stride_l, qC_stride_g;
  const float* B_scale;      /* (G,) */
  const float* C_scale;      /* (G,) */
  const int8_t* D;           /* (H,) or (H,P) int8, or NULL */
  int64_t D_stride_h;
  int32_t D_has_hdim;
  const float* D_scale;      /* device scalar */
  const float* state_scale;  /* (H,P) view: static_state_scale */
  int64_t ss_stride_h, ss_stride_p;
  const float* cb_scale;     /* (G,): static_cb_scale */
  const float* alpha_hp;     /* value side: (H,P) view */
  int64_t alpha_stride_h, alpha_stride_p;
  const float* bscale_g;     /* value side: (G,) */
  int64_t bscale_stride_g;
  const float* x_scale_hp;   /* key side: (H,P) view */
  int64_t xs_stride_h, xs_stride_p;
  const float* b_gate_scale; /* key side: 4-D broadcastable (B,nc,H,N) */
  int64_t bgs_stride_b, bgs_stride_c, bgs_stride_h, bgs_stride_n;
  int32_t keyside;
  int32_t gate_shift;        /* fractional bits of the state-passing gate (reference: 7) */
  void* out;                 /* (B,L,H,P) fp16 contiguous */
  int8_t* final_states;      /* (B,H,P*N) int8 contiguous, or NULL */
  void* workspace;           /* device memory, 256-byte aligned, lq_ssd_combined_workspace_bytes() bytes; contents undefined
                                on entry and on return (ignored by lq_ssd_combined_static) */
  int64_t workspace_bytes;
  int32_t batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size;
  const float* b_rowmax;     /* key side, optional: (B,L,G) fp32 max_n |b_fp| per token row as lq_split_rotate_quant_xBC
                                writes it beside b_fp; NULL: the call computes it into the workspace */
} lq_ssd_combined_args;
int lq_ssd_combined(const lq_ssd_combined_args* args, hipStream_t stream);
/* workspace size for the dims in `args` (pointers are not read), written to *bytes */
int lq_ssd_combined_workspace_bytes(const lq_ssd_combined_args* args, int64_t* bytes);

/* No counterpart in the reference.  lq_ssd_combined for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid it): the intermediates live in a device array of
 * LQ_SSD_STATIC_WORKSPACE_BYTES that is part of the library image (one per GPU, held until the process ends), so the
 * call takes inputs and outputs only (`workspace` is ignored) and allocates nothing.  Returns LQ_E_SHAPE when the dims
 * need more than that.  Every call on one GPU shares the array: calls that overlap on one GPU race (serialize them on
 * one stream or with events); nothing in it needs clearing between calls, every byte a stage reads was written by an
 * earlier stage of the same call.  A graph that captured this call replays into the same array: replays race with any
 * other call of this entry on that GPU unless the caller orders them.
 * The array's device address is looked up once per GPU, by lq_ssd_static_init() or by the first call on that GPU; the
 * look-up never runs on a stream that is being captured: such a call returns LQ_E_STATE when no earlier eager call or
 * lq_ssd_static_init() (with that device current) has done it. */
#define LQ_SSD_STATIC_WORKSPACE_BYTES (64ll << 20)
int lq_ssd_combined_static(const lq_ssd_combined_args* args, hipStream_t stream);
/* No counterpart in the reference.  Set-up of lq_ssd_combined_static for the current device (idempotent, launches nothing). */
int lq_ssd_static_init(void);

/* ------------------------------------------------------------------------------------------
 * Rotation + quantize prologue.
 * ------------------------------------------------------------------------------------------ */

/* replaces fused_split_rotate_quant_xBC, linquant/kernels/mamba2/fused_split_rotate_xBC.py:236-329
 * (kernel :31-227): B and C lanes of xBC -> [*dqk, fp16] -> signs -> H2 (x) H_{N/2} -> fp16 ->
 * clamp(rint(y*inv_scale), -128, 127).  x is returned by the caller as a view, never touched here. */
typedef struct {
  const void* xBC;           /* (B,T,d_ssm+2*G*N) fp16, unit last stride */
  int64_t xBC_stride_b, xBC_stride_t;
  int8_t* qB;                /* (B,T,G,N) int8 contiguous */
  int8_t* qC;                /* (B,T,G,N) int8 contiguous */
  void* b_fp;                /* NULL, or (B,T,G,N) fp16 contiguous: the rotated fp16 B (what q_B is quantized from), i.e.
                                kronecker_hadamard_fwd of the [dqk-scaled] B lanes, for the key-side chunk state */
  const void* signs;         /* (G,N) +-1 values of dtype signs_dtype, or NULL for no rotation */
  int32_t signs_dtype;       /* LQ_DT_F16 / LQ_DT_F32 / LQ_DT_I8 */
  const float* B_inv_scale;  /* (G,) */
  const float* C_inv_scale;  /* (G,) */
  const float* dqk_b;        /* (G*N,) fp32 holding fp16-rounded values, or NULL */
  const float* dqk_c;
  int32_t batch, seqlen, d_ssm, ngroups, dstate;
  float* b_rowmax;           /* NULL, or (B,T,G) fp32: max_n |b_fp[b,t,g,n]| per token row (needs b_fp), the table the
                                key-side chunk state uses to leave out all-zero slabs (its b_rowmax with b_rowmax_ready) */
} lq_split_rotate_quant_xBC_args;
int lq_split_rotate_quant_xBC(const lq_split_rotate_quant_xBC_args* args, hipStream_t stream);

/* replaces kronecker_hadamard_fwd, linquant/kernels/hadamard.py:141-179 (kernel :38-103):
 * y = (x * signs) . (H2 (x) H_{D/2}) per head, same dtype out, no quantization. */
typedef struct {
  const void* x;             /* (B,T,H,D) fp16 or bf16 (x_dtype), unit D stride; D a power of two, 64 .. 512 */
  int64_t x_stride_b, x_stride_t, x_stride_h;
  void* y;                   /* (B,T,H,D) contiguous, same dtype as x */
  const void* signs;         /* (H,D) */
  int32_t signs_dtype;
  int32_t batch, seqlen, nheads, dim;
  int32_t x_dtype;           /* LQ_DT_F16 (0) or LQ_DT_BF16 */
} lq_kron_hadamard_args;
int lq_kron_hadamard(const lq_kron_hadamard_args* args, hipStream_t stream);

/* ------------------------------------------------------------------------------------------
 * Zoo chunk kernels: linear attention (no / scalar decay), GLA, DeltaNet / Gated DeltaNet, KDA.
 * q,k (B,T,H,K) and v (B,T,H,V) fp16/bf16 contiguous, T a multiple of the chunk size, K in {64,128},
 * V a multiple of 64.  The chunk size is 64; every entry point but lq_zoo_rotate_quant also takes 128 (the kernels then
 * walk a chunk as two 64-token halves; see each entry).  g holds the chunk-local cumulative log decay (lq_zoo_cumsum).  Scales are
 * fp32: q,k,w (H,), kw (H,K), vw,vl,el,ew,state (H,V).  h_i8 is the per-chunk INT8 stored state in
 * V-major layout (B,NT,H,V,K): an internal buffer shared by the state and output kernels.
 * qmax is 127 (INT8) or 31 (INT6 codes in INT8 containers); the stored state always uses 127.
 * ------------------------------------------------------------------------------------------ */

/* replaces the torch prep of the zoo wrappers: chunk-local fp32 cumsum of g and the log envelope
 * (linquant/kernels/zoo/simple_gla.py:191, gla.py:249-251, gated_delta_rule.py:174, kda.py:168-170) */
typedef struct {
  const float* g;            /* (B,T,H) or (B,T,H,K) fp32 contiguous */
  float* gc;                 /* same shape */
  float* logenv;             /* (B,T,H) max_k(gc_last[k] - gc[t,k]); diagonal decay only, else NULL */
  int32_t batch, seqlen, nheads, kdim; /* kdim = 0: scalar decay */
  int32_t chunk_size;        /* scalar decay: any divisor of seqlen; per-channel decay: a multiple of 16 up to 64, or 128 */
  /* Optional (per-channel decay, linear family, chunk 64; all of them when kqT is set): the write operands of the state
   * kernel that lq_zoo_write_codes would make from gc and logenv, made here while the chunk's decay tile is on chip:
   * the operand preparation inside _gla_state_body (linquant/kernels/zoo/gla.py:124-141).  Same bits. */
  const void* k;             /* (B,T,H,K) fp16/bf16 */
  const void* v;             /* (B,T,H,V) fp16/bf16 */
  int8_t* kqT;               /* (B,NT,H,K,C) key write codes */
  int8_t* vqT;               /* (B,NT,H,V,C) value write codes */
  float* ev;                 /* (B,T,H) */
  float* gam;                /* (B,NT,H,K) */
  const float* skw;          /* (H,K) */
  const float* svw;          /* (H,V) */
  float eta;
  int32_t qmax;
  int32_t vdim;
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16 */
} lq_zoo_cumsum_args;
int lq_zoo_cumsum(const lq_zoo_cumsum_args* args, hipStream_t stream);

#define LQ_FAMILY_LINEAR 0
#define LQ_FAMILY_DELTA 1
#define LQ_DECAY_NONE 0
#define LQ_DECAY_SCALAR 1
#define LQ_DECAY_DIAGONAL 2

/* replaces the operand preparation inside the reference's state kernels (linquant/kernels/zoo/simple_gla.py:55-66,
 * gla.py:124-141, gated_delta_rule.py:85-105, kda.py:100-124): every write operand that does not depend on the
 * carried state is quantized once, in parallel over chunks, into the layout lq_zoo_state consumes.
 * kqT/vqT are channel-major inside each 64-token chunk; all five outputs are internal buffers of the wrappers.
 * chunk_size is 64, or 128 (linear family with no / scalar decay: also 192, 256; seqlen a multiple of it): the buffers keep
 * their 64-token layout (NT = seqlen / 64) and the decays of a chunk's earlier tokens reach on to the end of the chunk. */
typedef struct {
  const void* key;           /* key operand of the write: k (linear) or Hw (delta), (B,T,H,K) fp16/bf16 */
  const void* val;           /* linear family: v (B,T,H,V) fp16/bf16; delta family: NULL */
  const void* w;             /* delta family: W (B,T,H,K) fp16/bf16; linear family: NULL */
  const float* g;            /* cumulative log decay (B,T,H) / (B,T,H,K), or NULL for no decay */
  const float* logenv;       /* diagonal decay: (B,T,H) */
  int8_t* kqT;               /* (B,NT,H,K,64) int8 key write codes */
  int8_t* vqT;               /* (B,NT,H,V,64) int8 value write codes (linear family) */
  int8_t* wq;                /* (B,T,H,K) int8 state-read codes of W (delta family) */
  float* ev;                 /* (B,T,H) fp32 value-side decay factor of each token */
  float* gam;                /* (B,NT,H,K) fp32 chunk decay of each state row */
  const float* skw;          /* (H,K) key write scale */
  const float* svw;          /* (H,V) value write scale (linear family) */
  const float* sw;           /* (H,) W scale (delta family) */
  float eta;
  int32_t qmax;
  int32_t batch, seqlen, nheads, kdim, vdim, chunk_size;
  int32_t decay;
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16: dtype of every 16-bit activation tensor of the call */
} lq_zoo_write_codes_args;
int lq_zoo_write_codes(const lq_zoo_write_codes_args* args, hipStream_t stream);

/* replaces the chunk loops of _state_kernel (linquant/kernels/zoo/simple_gla.py:23-95), _gla_state_kernel
 * (gla.py:102-167), _delta_state_kernel (gated_delta_rule.py:50-136) and _kda_state_kernel (kda.py:68-151):
 * sequential chunk loop with an fp32 carry, INT8 stored copy per chunk, INT8 write product (and, delta family,
 * the INT8 state read W.S and the pseudo-values E = (U - W.S) * fw, stored fp16 for the output kernel).
 * Consumes the buffers written by lq_zoo_write_codes.
 * chunk_size is 64, or 128 (operands from lq_zoo_write_codes with chunk_size 128, delta family: W and U
 * from lq_zoo_wy_prep with chunk_size 128): one stored state per 128 tokens, h_i8 is (B,seqlen/128,H,V,K), both halves of
 * a chunk read it, and the carry takes the INT8 write product summed over the 128 tokens (int32) once per chunk.  The linear
 * family in rotated storage also takes 192 and 256 (h_i8 (B,seqlen/chunk_size,H,V,K)). */
typedef struct {
  const int8_t* kqT;         /* (B,NT,H,K,64) */
  const int8_t* vqT;         /* linear family: (B,NT,H,V,64) */
  const int8_t* wq;          /* delta family: (B,T,H,K) */
  const void* u;             /* delta family: U (B,T,H,V) fp16/bf16 */
  const float* fw;           /* delta family: (B,T,H) fp32 value-side share of the outer beta factor */
  const float* ev;           /* delta family: (B,T,H) */
  const float* gam;          /* (B,NT,H,K) */
  int8_t* h_i8;              /* (B,NT,H,V,K) int8 */
  void* e_out;               /* delta family: (B,T,H,V) fp16/bf16 */
  float* ht;                 /* (B,H,K,V) fp32 final carry, or NULL */
  const float* skw;          /* (H,K) key write scale */
  const float* svw;          /* (H,V) value write scale: vw (linear) or ew (delta) */
  const float* sw;           /* (H,) W scale (delta) */
  const float* ss;           /* (H,V) state scale */
  const void* unrot;         /* (V,V) fp16 R_V^T for canonical storage, or NULL */
  int32_t qmax;
  int32_t batch, seqlen, nheads, kdim, vdim, chunk_size;
  int32_t family;
  int32_t vtile;             /* value columns per workgroup: 16, 32, 64, or 0 = chosen from the grid size */
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16: dtype of every 16-bit activation tensor of the call */
  /* Optional (delta family): fw, ev and gam once more, packed per (batch, chunk, head) as 64 + 64 + K consecutive floats
   * (what lq_zoo_wy_prep writes into its `pack`): the kernel then fetches a chunk's per-token factors and row decays
   * from three contiguous pieces instead of 64 addresses 4 H bytes apart.  NULL: fw, ev and gam are read. */
  const float* pack;         /* (B,NT,H,128+K) fp32 or NULL */
} lq_zoo_state_args;
int lq_zoo_state(const lq_zoo_state_args* args, hipStream_t stream);

/* replaces _output_kernel (linquant/kernels/zoo/simple_gla.py:98-172) and _gla_output_kernel
 * (gla.py:170-232): o = dequant(q8(q).h_i8) [* exp(g)] + (fp16(A) . fp16(q8(v))) * svl, with A computed
 * in-kernel from q8(q).q8(k)^T (no / scalar decay) or read from the fp32 A tensor (diagonal decay).
 * chunk_size is 64, or 128 (raw q, k, v; h_i8 (B,seqlen/128,H,V,K) from lq_zoo_state with chunk_size
 * 128; under diagonal decay A and A_cross from lq_zoo_gla_A with chunk_size 128): two launches, the first leaves the
 * second halves' products with the first halves' tokens in `cross`, the second starts its fp32 accumulators from them.
 * No / scalar decay in rotated storage also takes 192 and 256 (one such launch per earlier 64-token piece). */
typedef struct {
  const void* q;             /* no / scalar decay: (B,T,H,K) fp16/bf16; diagonal decay: NULL */
  const int8_t* qg;          /* diagonal decay: (B,T,H,K) int8 codes of q*exp(g)*scale written by lq_zoo_gla_A */
  const void* k;             /* no / scalar decay: k or Hw (B,T,H,K) fp16/bf16; diagonal: NULL */
  const void* v;             /* local value operand: v or e_out (B,T,H,V) fp16/bf16 */
  const int8_t* h_i8;        /* (B,NT,H,V,K) */
  const float* g;            /* cumulative log decay or NULL */
  const void* A;             /* diagonal decay: (B,T,H,C) fp16 lower-triangular intra-chunk product */
  void* o;                   /* (B,T,H,V) fp16/bf16, or fp32 when o_is_f32 */
  int32_t o_is_f32;
  const float* sq;           /* (H,) */
  const float* sk;           /* (H,) (no / scalar decay) */
  const float* svl;          /* (H,V), 16-byte aligned */
  const float* ss;           /* (H,V), 16-byte aligned */
  const void* unrot;         /* (V,V) fp16 or NULL */
  float scale;
  int32_t qmax;
  int32_t batch, seqlen, nheads, kdim, vdim, chunk_size;
  int32_t decay;
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16: dtype of every 16-bit activation tensor of the call */
  /* Optional (no / scalar decay, rotated storage): the local codes of q, k and v ready-made by lq_zoo_rotate_quant;
   * q, k, v are then not read (may be NULL) and nothing is quantized here. */
  const int8_t* qc;          /* (B,T,H,K) int8 q8(q*scale, 1/sq) */
  const int8_t* kc;          /* (B,T,H,K) int8 q8(k, 1/sk) */
  const int8_t* vc;          /* (B,T,H,V) int8 q8(v, 1/svl) */
  float* cross;              /* chunk_size above 64: (B,T,H,V) fp32 workspace, 16-byte aligned (overwritten); else unused */
  const void* A_cross;       /* chunk_size 128, diagonal decay: (B,T,H,64) fp16 written by lq_zoo_gla_A; else unused */
} lq_zoo_output_args;
int lq_zoo_output(const lq_zoo_output_args* args, hipStream_t stream);

/* replaces chunk_simple_gla_int8 as a whole (linquant/kernels/zoo/simple_gla.py:175-212; rotated storage, raw operands):
 * lq_zoo_cumsum (scalar decay only), lq_zoo_write_codes, lq_zoo_state and lq_zoo_output launched back to back on `stream`
 * over one caller-supplied workspace that holds the intermediates (cumulative decay, write codes, per-token factors, stored
 * states, and for chunk sizes above 64 the cross workspace).  Same kernels and bits as the four calls; one foreign call and
 * one allocation per forward, which is what bounds small shapes.  Field meanings as in the per-stage structs. */
typedef struct {
  const void* q;             /* (B,T,H,K) fp16/bf16 */
  const void* k;             /* (B,T,H,K) */
  const void* v;             /* (B,T,H,V) */
  const float* g;            /* (B,T,H) fp32 log decay per token (not cumulated), or NULL: no decay */
  void* o;                   /* (B,T,H,V) fp16/bf16, or fp32 when o_is_f32 */
  int32_t o_is_f32;
  float* ht;                 /* (B,H,K,V) fp32 final state, or NULL */
  const float* sq;           /* (H,) */
  const float* sk;           /* (H,) */
  const float* skw;          /* (H,K) */
  const float* svw;          /* (H,V) */
  const float* svl;          /* (H,V), 16-byte aligned */
  const float* ss;           /* (H,V), 16-byte aligned */
  float eta, scale;
  int32_t qmax;
  int32_t batch, seqlen, nheads, kdim, vdim, chunk_size; /* K in {64,128}, V a multiple of 64, chunk 64, 128, 192 or 256 */
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16 */
  void* workspace;           /* device memory, 256-byte aligned, lq_zoo_simple_gla_workspace_bytes() bytes; contents undefined
                                on entry and on return */
  int64_t workspace_bytes;
} lq_zoo_simple_gla_args;
int lq_zoo_simple_gla(const lq_zoo_simple_gla_args* args, hipStream_t stream);
/* workspace size for the dims in `args` (pointers are not read), written to *bytes */
int lq_zoo_simple_gla_workspace_bytes(const lq_zoo_simple_gla_args* args, int64_t* bytes);

/* replaces chunk_gla_int8 (linquant/kernels/zoo/gla.py:235-279), chunk_delta_int8 (gated_delta_rule.py:159-203) and
 * chunk_kda_int8 (kda.py:154-203) as a whole (rotated storage): the stage entry points above in the order the wrappers
 * issue them -- cumsum, WY prep (delta family), write-codes pre-pass (128-token chunks; 64-token chunks make them in the
 * cumsum / WY launch), A kernel (per-channel decay), state recurrence, output -- on `stream` over one caller-supplied
 * workspace that holds every intermediate.  Same kernels and bits as the separate calls; one foreign call and one
 * allocation per forward.  family x decay: linear x diagonal = GLA; delta x none = DeltaNet, delta x scalar = Gated
 * DeltaNet, delta x diagonal = KDA (linear x none / scalar: lq_zoo_simple_gla).  Field meanings as in the per-stage structs. */
typedef struct {
  const void* q;             /* (B,T,H,K) fp16/bf16 */
  const void* k;             /* (B,T,H,K) */
  const void* v;             /* (B,T,H,V) */
  const float* g;            /* log decay per token, not cumulated: (B,T,H) scalar, (B,T,H,K) diagonal, NULL none */
  const float* beta;         /* delta family: (B,T,H) fp32 */
  void* o;                   /* (B,T,H,V) fp16/bf16, or fp32 when o_is_f32 */
  int32_t o_is_f32;
  float* ht;                 /* (B,H,K,V) fp32 final state, or NULL */
  const float* sq;           /* (H,) */
  const float* sk;           /* (H,) */
  const float* sw;           /* delta family: (H,) */
  const float* skw;          /* (H,K) */
  const float* svw;          /* (H,V) value write scale: vw (linear) or ew (delta) */
  const float* svl;          /* (H,V) local value scale: vl (linear) or el (delta); 16-byte aligned */
  const float* ss;           /* (H,V), 16-byte aligned */
  const void* rot;           /* diagonal decay: (K,K) fp16 local R_QK, or NULL */
  const float* dq;           /* KDA, 64-token chunks: (H,K) D_QK applied to q and k as they are loaded, or NULL */
  const float* dq_rcp;       /* (H,K) RN(1 / dq), with dq */
  float sigma, tau, eta, scale;
  int32_t qmax;
  int32_t family, decay;
  int32_t batch, seqlen, nheads, kdim, vdim, chunk_size; /* K in {64,128}, V a multiple of 64, chunk 64 or 128 */
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16 */
  void* workspace;           /* device memory, 256-byte aligned, lq_zoo_chunk_forward_workspace_bytes() bytes; contents
                                undefined on entry and on return */
  int64_t workspace_bytes;
} lq_zoo_chunk_forward_args;
int lq_zoo_chunk_forward(const lq_zoo_chunk_forward_args* args, hipStream_t stream);
/* workspace size for the dims, family, decay and chunk size in `args` (pointers are not read), written to *bytes */
int lq_zoo_chunk_forward_workspace_bytes(const lq_zoo_chunk_forward_args* args, int64_t* bytes);

/* replaces _gla_A_inter + _gla_A_intra (linquant/kernels/zoo/gla.py:27-99): intra-chunk product under
 * per-channel decay, 16-token sub-blocks: INT8 dots on anchor-rescaled operands off the diagonal, fp32
 * reduction over the dequantized codes on the diagonal blocks.  Writes the full (C,C) rows (C = 64; chunk_size 128:
 * two (64,64) tensors, see A_cross), zeros above
 * the diagonal, and the INT8 codes of the decayed query (gla.py:188-190 computes them in the output kernel). */
typedef struct {
  const void* q;             /* (B,T,H,K) fp16/bf16 */
  const void* k;             /* (B,T,H,K) fp16/bf16: k (GLA) or Hw (KDA) */
  const float* g;            /* (B,T,H,K) cumulative log decay */
  void* A;                   /* (B,T,H,C) fp16: the fp32 product rounded once, as the local product consumes it */
  int8_t* qg;                /* (B,T,H,K) int8 codes q8(q*exp(g)*scale, 1/sq): the state-read operand of the output kernel */
  const void* rot;           /* (K,K) fp16 local R_QK, or NULL */
  const float* sq;
  const float* sk;
  float scale;
  int32_t qmax;
  int32_t batch, seqlen, nheads, kdim, chunk_size;
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16: dtype of every 16-bit activation tensor of the call */
  const float* dq;           /* optional (H,K) fp32 D_QK (linquant/harness.py:68-88) applied to q as it is loaded:
                                q' = act(q * dq), exactly what lq_zoo_rotate_qkv would have stored; NULL: q as it is */
  void* A_cross;             /* chunk_size 128 (g cumulated over 128 tokens): (B,T,H,64) fp16; rows of the second halves
                                receive their blocks with the first halves' tokens (column j = token j of the chunk), A
                                the blocks inside either half, as for chunk_size 64; else unused */
} lq_zoo_gla_A_args;
int lq_zoo_gla_A(const lq_zoo_gla_A_args* args, hipStream_t stream);

/* replaces the WY / UT prep of the delta family (linquant/kernels/zoo/gated_delta_rule.py:20-47 and
 * kda.py:22-53; the reference's default sigma=tau=1 route through fla-core's prep kernels is replaced by
 * the same native prep): fp32 Gram with decay, unit-lower-triangular inverse, W = T.(L*exp(g)),
 * U = T.(beta^sigma v), Hw = beta^((1-sigma)tau) k, fw = beta^((1-sigma)(1-tau)).
 * chunk_size is 64, or 128 (g cumulated over 128 tokens; 128 x 128 Gram matrix and inverse in a kernel of its own,
 * which stores Hw, W, U, fw only: kqT, dk_div and pack must be NULL, lq_zoo_write_codes makes the write codes). */
typedef struct {
  const void* k;             /* (B,T,H,K) fp16/bf16 */
  const void* v;             /* (B,T,H,V) fp16/bf16 */
  const float* beta;         /* (B,T,H) fp32 */
  const float* g;            /* cumulative log decay (B,T,H) / (B,T,H,K) or NULL */
  void* Hw;                  /* (B,T,H,K) fp16/bf16 */
  void* W;                   /* (B,T,H,K) fp16/bf16; may be NULL when the codes below are requested */
  void* U;                   /* (B,T,H,V) fp16/bf16 */
  float* fw;                 /* (B,T,H) fp32 */
  float sigma, tau;
  int32_t batch, seqlen, nheads, kdim, vdim, chunk_size;
  int32_t decay;
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16: dtype of every 16-bit activation tensor of the call */
  /* Optional (all of them when kqT is set): the write-operand codes lq_zoo_write_codes would make from the stored Hw
   * and W, made here from the same rounded values (same bits), so that the state kernel needs no pre-pass of its own
   * and W need not be stored: operand preparation inside _delta_state_body (gated_delta_rule.py:85-105) and
   * _kda_state_body (kda.py:100-124). */
  int8_t* kqT;               /* (B,NT,H,K,C) int8 key write codes, channel-major inside the chunk */
  int8_t* wq;                /* (B,T,H,K) int8 state-read codes of W */
  float* ev;                 /* (B,T,H) per-token value factor */
  float* gam;                /* (B,NT,H,K) per-channel chunk decay */
  const float* logenv;       /* (B,T,H) log envelope (per-channel decay) */
  const float* skw;          /* (H,K) key write scales */
  const float* sw;           /* (H,) state-read scale of W */
  float eta;
  int32_t qmax;
  /* Optional D_QK (linquant/harness.py:68-88) applied to k as it is loaded: k' = act(k / dk_div), the quotient rounded
   * once, exactly what lq_zoo_rotate_qkv would have stored; both NULL: k is used as it is.  Taken only together with the
   * write-operand codes above (kqT set). */
  const float* dk_div;       /* (H,K) fp32 D_QK, finite and positive */
  const float* dk_rcp;       /* (H,K) fp32 RN(1 / dk_div) */
  /* Optional, with the write-operand codes: fw, ev and gam once more, packed per (batch, chunk, head) as 64 + 64 + K
   * consecutive floats, the layout lq_zoo_state reads a chunk's factors from in three contiguous pieces. */
  float* pack;               /* (B,NT,H,128+K) fp32 or NULL */
} lq_zoo_wy_prep_args;
int lq_zoo_wy_prep(const lq_zoo_wy_prep_args* args, hipStream_t stream);

/* replaces the operand rotations in front of a zoo call: the three GEMMs q @ R_QK, k @ R_QK, v @ R_V of
 * bench/zoo_kernels.py:135-140 (the oracle's entry rotation, linquant/reference.py:42-46) and the diagonal q / k
 * rescaling D_QK of linquant/harness.py:68-88, in one launch:
 *   q_out = act((q * dq) . H_K / sqrt(K) * signs_qk),  k_out likewise with k / dq,  v_out = act(v . H_V / sqrt(V) * signs_v)
 * with the Sylvester Hadamard matrix H_n (linquant/reference.py:232-239: R = H_n / sqrt(n) . diag(signs)), evaluated as a
 * fast Walsh-Hadamard transform in fp32 and rounded once to the activation dtype.  A tensor whose input pointer is NULL
 * is skipped; NULL signs leave out the rotation (diagonal-decay cells rotate locally inside lq_zoo_gla_A); NULL dq / dk
 * leave out the rescaling.  In place (q_out == q) is allowed. */
typedef struct {
  const void* q;             /* (B,T,H,K) fp16/bf16 contiguous, or NULL */
  const void* k;             /* (B,T,H,K), or NULL */
  const void* v;             /* (B,T,H,V), or NULL */
  void* q_out;               /* same shape and dtype as the input */
  void* k_out;
  void* v_out;
  const float* dq;           /* (H,K) fp32 D_QK, finite and positive: q is multiplied by it, k divided (the quotient is
                                rounded once to fp32, as the float64 division of harness.py:86 rounds); or NULL */
  const float* dk;           /* (H,K) fp32 RN(1 / dq), set exactly when k is to be rescaled (needs dq), or NULL */
  const float* signs_qk;     /* (K,) fp32 +-1 column signs of R_QK, or NULL */
  const float* signs_v;      /* (V,) fp32 +-1 column signs of R_V, or NULL */
  int32_t batch, seqlen, nheads, kdim, vdim; /* kdim, vdim in {64, 128} */
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16 */
} lq_zoo_rotate_qkv_args;
int lq_zoo_rotate_qkv(const lq_zoo_rotate_qkv_args* args, hipStream_t stream);

/* replaces, for the linear family under no / scalar decay, the same operand prologue (bench/zoo_kernels.py:135-140, "not
 * fused yet"; linquant/harness.py:68-88) TOGETHER WITH the operand quantization it feeds: the write-operand preparation
 * inside _state_body (linquant/kernels/zoo/simple_gla.py:55-66) and the code loop at the top of _output_body
 * (simple_gla.py:125-140).  One launch reads q, k, v once and emits every INT8 operand of lq_zoo_state and lq_zoo_output;
 * each code equals what lq_zoo_rotate_qkv -> lq_zoo_write_codes / lq_zoo_output would have made from the rotated
 * activations stored in between (same arithmetic on the same rounded values).  q_out / k_out / v_out are optional. */
typedef struct {
  const void* q;             /* (B,T,H,K) fp16/bf16 contiguous */
  const void* k;             /* (B,T,H,K) */
  const void* v;             /* (B,T,H,V) */
  void* q_out;               /* rotated / rescaled activations, same shape and dtype; NULL: not stored */
  void* k_out;
  void* v_out;
  int8_t* qc;                /* (B,T,H,K) local codes q8(q'*scale, 1/sq) */
  int8_t* kc;                /* (B,T,H,K) local codes q8(k', 1/sk) */
  int8_t* vc;                /* (B,T,H,V) local codes q8(v', 1/svl) */
  int8_t* kqT;               /* (B,NT,H,K,C) key write codes q8(k'*fk, 1/skw), channel-major inside the chunk */
  int8_t* vqT;               /* (B,NT,H,V,C) value write codes q8(v'*fv, 1/svw) */
  float* ev;                 /* (B,T,H) per-token value factor fv */
  float* gam;                /* (B,NT,H,K) chunk decay */
  const float* dq;           /* (H,K) D_QK or NULL (see lq_zoo_rotate_qkv) */
  const float* dk;           /* (H,K) RN(1 / dq), set exactly when k is to be rescaled, or NULL */
  const float* signs_qk;     /* (K,) +-1 column signs of R_QK, or NULL */
  const float* signs_v;      /* (V,) +-1 column signs of R_V, or NULL */
  const float* g;            /* (B,T,H) chunk-local cumulative log decay (scalar decay), or NULL */
  const float* sq;           /* (H,) */
  const float* sk;           /* (H,) */
  const float* svl;          /* (H,V) */
  const float* skw;          /* (H,K) */
  const float* svw;          /* (H,V) */
  float eta, scale;
  int32_t qmax;
  int32_t batch, seqlen, nheads, kdim, vdim, chunk_size; /* kdim, vdim in {64, 128}; chunk 64 */
  int32_t act_dtype;         /* LQ_DT_F16 or LQ_DT_BF16 */
} lq_zoo_rotate_quant_args;
int lq_zoo_rotate_quant(const lq_zoo_rotate_quant_args* args, hipStream_t stream);

/* ------------------------------------------------------------------------------------------
 * Element-wise stages in front of the Mamba-2 SSD prologue.
 * ------------------------------------------------------------------------------------------ */

/* replaces _fused_fp16_to_int8 (linquant/w4a8_linear.py:36-98): q = clamp(rint(x * (1/s)) or rint(x / s), clamp_min, 127) */
typedef struct {
  const void* x;             /* (M,N) fp16, unit column stride */
  int64_t x_stride;          /* row stride in elements */
  int8_t* out;               /* (M,N) int8 contiguous */
  const void* scale;         /* device scalar */
  int32_t scale_dtype;       /* LQ_DT_F16 / LQ_DT_F32 */
  int32_t rows, cols;        /* cols a multiple of 8 */
  float clamp_min;           /* -127 (default) or -128 */
  int32_t reciprocal;        /* 1: x * (1/s);  0: IEEE x / s */
} lq_fp16_to_int8_args;
int lq_fp16_to_int8(const lq_fp16_to_int8_args* args, hipStream_t stream);

/* replaces causal_conv1d_fn(x, weight, bias, activation="silu") of causal-conv1d==1.5.3.post1 as called at
 * linquant/quantized_mamba2.py:262-268 (channel-last layout, no initial state) */
typedef struct {
  const void* x;             /* (B,L,D) fp16, unit D stride */
  int64_t x_stride_b, x_stride_l;
  const void* weight;        /* (D,W) fp16 contiguous, 16-byte aligned */
  const void* bias;          /* (D,) fp16 or NULL, 16-byte aligned */
  void* out;                 /* (B,L,D) fp16 contiguous */
  int32_t batch, seqlen, dim, width; /* dim a multiple of 8, width 2..4 */
  int32_t silu;              /* 1: SiLU activation, 0: none */
} lq_causal_conv1d_args;
int lq_causal_conv1d(const lq_causal_conv1d_args* args, hipStream_t stream);

/* ------------------------------------------------------------------------------------------
 * Stages behind the Mamba-2 SSD: gated RMSNorm and the Hadamard + INT8 quantizer of the out_proj input.
 * ------------------------------------------------------------------------------------------ */

/* replaces `self.norm(y, z)` at linquant/quantized_mamba2.py:354-358 (RMSNormGated with norm_before_gate = False and
 * group_size = d_ssm / ngroups; the gate stays fp16):
 *   v = x * (z * sigmoid(z));  out = fp16(v * rsqrt(mean_group(v^2) + eps) * weight), all in fp32 */
typedef struct {
  const void* x;             /* (rows, dim) fp16, unit column stride */
  int64_t x_stride;          /* row stride in elements, a multiple of 8 */
  const void* z;             /* gate, (rows, dim) fp16, or NULL for a plain RMSNorm */
  int64_t z_stride;
  const void* weight;        /* (dim,) */
  int32_t weight_dtype;      /* LQ_DT_F16 / LQ_DT_F32 */
  void* out;                 /* (rows, dim) fp16 contiguous */
  int32_t rows, dim;         /* dim = 128 * g, g <= 64 */
  int32_t group_size;        /* divides dim, a multiple of 8 */
  float eps;
} lq_rmsnorm_gated_args;
int lq_rmsnorm_gated(const lq_rmsnorm_gated_args* args, hipStream_t stream);

/* replaces qhad_transform (linquant/hadamard_utils.py:9-19), i.e. the fast_hadamard_transform_{12N,20N,28N,40N,pow2}
 * kernels with INT8 output: q = clamp(round_half_away((H x) * scale), -127, 127) per row, H = had (x) H_128:
 * the row is cut into g = dim / 128 contiguous chunks; chunk c' of H x is sum_c had[c'][c] * H_128 chunk_c with the
 * Sylvester H_128.  For dim = m * 2^k, had = H_m (x) Sylvester H_(2^k / 128). */
typedef struct {
  const void* x;             /* (rows, dim) fp16, unit column stride */
  int64_t x_stride;          /* row stride in elements, a multiple of 8 */
  const int8_t* had;         /* (g, g) entries +1 / -1, row-major */
  int8_t* out;               /* (rows, dim) int8 contiguous */
  int32_t rows, dim;         /* dim = 128 * g, g <= 64 */
  float scale;               /* had_scale / input_scale = 1 / (sqrt(dim) * input_scale) */
} lq_qhad_transform_args;
int lq_qhad_transform(const lq_qhad_transform_args* args, hipStream_t stream);

/* the two stages above in one launch (linquant/quantized_mamba2.py:354-364 when d_mlp = 0): the normalized row is
 * rounded to fp16 exactly as the separate stages would store it, but never leaves the compute unit */
typedef struct {
  const void* x;             /* as in lq_rmsnorm_gated_args */
  int64_t x_stride;
  const void* z;
  int64_t z_stride;
  const void* weight;
  int32_t weight_dtype;
  void* norm_out;            /* NULL, or (rows, dim) fp16 contiguous: the normalized rows are stored as well */
  int32_t rows, dim, group_size;
  float eps;
  const int8_t* had;         /* as in lq_qhad_transform_args */
  int8_t* out;
  float scale;
} lq_rmsnorm_gated_qhad_args;
int lq_rmsnorm_gated_qhad(const lq_rmsnorm_gated_qhad_args* args, hipStream_t stream);

/* ------------------------------------------------------------------------------------------
 * Calibration: running absolute maxima of an activation tensor, on the device.
 * ------------------------------------------------------------------------------------------ */

/* replaces the calibrating branch of Quantizer.__call__ (linquant/invariances.py:77-81):
 *   a = |x| [* gate];  a = amax over (batch, rows) keeping (H, D)  ("pc_static", mode 0)
 *                      | amax over (batch, rows, D) keeping (H)     ("ph_static", mode 1)
 *                      | amax over everything                        (per tensor,  mode 2)
 *   out = max(out, a)   -- the running maximum over calibration batches; the caller zero-fills `out` once
 * and the per-(H,P) / per-(H,N) SSD observers of scripts/nemotron_h_calibration.py (:293-345 x * scale_lut, :462-556
 * gated B broadcast from its group to the heads, :558-600 plain x): `gate` is an optional fp32 factor per (batch, row,
 * head) and `heads_per_group` > 1 reads x at head h / heads_per_group. */
typedef struct {
  const void* x;             /* (B, T, Hx, D) in any stride order, unit D stride; Hx = H / heads_per_group */
  int32_t x_dtype;           /* LQ_DT_F16 / LQ_DT_BF16 / LQ_DT_F32 */
  int64_t x_stride_b, x_stride_t, x_stride_h;
  const float* gate;         /* NULL or (B, T, H) fp32 with the strides below */
  int64_t gate_stride_b, gate_stride_t, gate_stride_h;
  float* out;                /* mode 0: (H, D); mode 1: (H,); mode 2: (1,); fp32, updated in place */
  int32_t batch, rows, nheads, dim, heads_per_group; /* dim a multiple of 8 */
  int32_t mode;
} lq_absmax_args;
int lq_absmax(const lq_absmax_args* args, hipStream_t stream);

/* replaces the chunk-state observer of scripts/nemotron_h_calibration.py:602-651, which wraps the unquantized
 * _chunk_state_fwd and keeps amax over (batch, chunk, N) of its fp32 result per (H, P):
 *   S[b,c,h][p][n] = sum_{k in chunk c} x[b,k,h,p] * gate[b,k,h] * B[b,k,h / heads_per_group,n]
 *   out[h][p] = max(out[h][p], max_{b,c,n} |S|)      (fp32 products and sums; the caller zero-fills `out` once)
 * gate = exp(dA_last - dA_k) * dt_k, fp32. */
typedef struct {
  const void* x;             /* (B,L,H,P) view, unit P stride */
  int32_t x_dtype;           /* LQ_DT_F16 / LQ_DT_BF16 / LQ_DT_F32 */
  int64_t x_stride_b, x_stride_l, x_stride_h;
  const void* B;             /* (B,L,G,N) view, unit N stride, 16-byte aligned rows */
  int32_t B_dtype;
  int64_t B_stride_b, B_stride_l, B_stride_g;
  const float* gate;         /* (B,L,H) fp32 view */
  int64_t gate_stride_b, gate_stride_l, gate_stride_h;
  float* out;                /* (H,P) fp32, updated in place */
  int32_t batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size; /* P a multiple of 64; N 64, 128 or 256 */
} lq_absmax_chunk_state_args;
int lq_absmax_chunk_state(const lq_absmax_chunk_state_args* args, hipStream_t stream);

/* replaces the C.B^T observer of scripts/nemotron_h_w4a8.py:126-169, which wraps the unquantized _bmm_chunk_fwd and
 * keeps amax over (batch, chunk, Q, Q) of its result per group:
 *   CB[b,c,g][m][k] = sum_n C[b,c*Q+m,g,n] * B[b,c*Q+k,g,n]     (every (m, k) pair of a chunk, not only k <= m)
 *   out[g] = max(out[g], max |CB|) */
typedef struct {
  const void* C;             /* (B,L,G,N) view, unit N stride, 16-byte aligned rows */
  int32_t C_dtype;
  int64_t C_stride_b, C_stride_l, C_stride_g;
  const void* B;
  int32_t B_dtype;
  int64_t B_stride_b, B_stride_l, B_stride_g;
  float* out;                /* (G,) fp32, updated in place */
  int32_t batch, seqlen, ngroups, dstate, chunk_size; /* N a multiple of 8 */
} lq_absmax_cb_args;
int lq_absmax_cb(const lq_absmax_cb_args* args, hipStream_t stream);

/* ------------------------------------------------------------------------------------------
 * Measurement aid (no counterpart in the reference): a matrix-core-only launch whose rate is the MFMA issue peak of
 * the machine, the denominator of the "fraction of INT8 MFMA peak" figures (the reference's metric is quoted against
 * the chip's INT8 peak; this measures it instead of assuming it).  Work per launch: blocks * 4 waves * iters * 8
 * instructions of 16x16x64 INT8 (32768 ops each) or 16x16x32 fp16 (16384 flops each), or blocks * 4 * iters * 4
 * instructions of 32x32x32 INT8 (65536 ops each).
 * ------------------------------------------------------------------------------------------ */
typedef struct {
  int32_t kind;              /* 0: i32 16x16x64 i8;  1: f32 16x16x32 f16;  2: i32 32x32x32 i8 */
  int32_t iters, blocks;
  int32_t* sink;             /* one device int, never written in practice */
} lq_probe_mfma_args;
int lq_probe_mfma(const lq_probe_mfma_args* args, hipStream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LINQUANT_HIP_H */
