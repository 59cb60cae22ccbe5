/* C ABI of one compiled kernel configuration ("config library").
 *
 * The autotuner turns every candidate configuration (tile sizes, wave count, LDS buffering, fuse
 * type) into its own shared object, exactly as the reference does, and binds it with ctypes.  Each
 * such library exports the symbols declared below for ONE operator; which operator is selected at
 * compile time by defining AAT_OP_ATTN, AAT_OP_RET, AAT_OP_RET_BWD, AAT_OP_ATTN_BWD or AAT_OP_RET_RECURRENT before
 * including this header
 * (the generated wrapper does that, so the compiler checks the definitions against this file).
 *
 * Conventions (same as the reference unless stated):
 *   - all tensors are contiguous row-major device buffers owned by the caller; nothing is allocated,
 *     freed or retained by the callee;
 *   - q [B,H,Seq_q,Kd], k [B,H,Seq_k,Kd], v [B,H,Seq_k,D], o/dO [B,H,Seq_q,D] are IEEE fp16;
 *     mask [H,Seq_q,Seq_k] fp16; r [B,H,Seq_q] fp32; dqaccum [B,H,Seq_q,Kd] fp32, zero on entry;
 *   - Kd, D and the tile shape are baked into the library (see config_string());
 *   - Seq_q must be a multiple of the library's Br and Seq_k of its Bc;
 *   - `profile*` launches the kernel repeatedly (one probe launch, then ceil(100 ms / t) launches) and
 *     returns the mean time of one launch in milliseconds, or -1 on any error;
 *   - `kernel_entry*` enqueues one launch and returns without synchronising.
 *
 * Differences from the reference, all additive:
 *   - the two reference-signature entry points keep the reference's argument ORDER, including the
 *     swapped (Seq_k, Seq_q) of kernel_entry, and its literal behaviour: softmax scale 0.125, no causal
 *     masking, null stream.  kernel_entry returns 0 on success (the reference always returns 0),
 *     a positive hipError_t on a launch failure, AAT_ERR_SHAPE for an indivisible shape;
 *   - the *_ex entry points take (Seq_q, Seq_k) in that order plus a runtime softmax scale, a causal
 *     flag, an optional workspace and the stream to launch on (a hipStream_t passed as void*);
 *   - workspace_size() says how many bytes of workspace a problem needs (attention forward: 0 unless the
 *     configuration splits the kv range; RetNet: the mask scan of AAT_MASK_SCAN, not needed by the other
 *     mask modes, and for a backward built with a stored dS the optional room for it); abi_version() and
 *     config_string() identify the library.
 */
#ifndef AAT_KERNEL_ABI_H
#define AAT_KERNEL_ABI_H

#include <stddef.h>

#define AAT_ABI_VERSION 4
#define AAT_ERR_SHAPE (-2)      /* Seq_q / Seq_k not divisible by the tile, or a non-positive size */
#define AAT_ERR_WORKSPACE (-3)  /* workspace missing or smaller than workspace_size() */
#define AAT_ERR_LIMIT (-4)      /* a valid shape beyond the fixed capacity of an entry point that cannot allocate */

/* Values of the `causal` argument of the RetNet *_ex entry points, whose mask is a tensor: how much of it
 * to walk.  Tiles in which the mask is zero contribute exactly nothing, so every mode gives the same bits. */
#define AAT_MASK_DENSE 0    /* every tile (what the reference does) */
#define AAT_MASK_CAUSAL 1   /* the caller promises mask == 0 above the diagonal: those tiles are skipped */
#define AAT_MASK_SCAN 2     /* the call first scans the mask (one read of it) into the workspace and then skips
                               the leading and trailing all-zero tiles of every band of rows; needs
                               workspace_size() bytes */
#define AAT_MASK_SCANNED 3  /* as AAT_MASK_SCAN, but the workspace already holds the scan of this same mask and
                               shape, written by an earlier AAT_MASK_SCAN call of any RetNet library */

typedef unsigned short aat_half; /* raw IEEE binary16 bits */

#ifdef __cplusplus
extern "C" {
#endif

/* Common to every config library. */
int abi_version(void);
const char* config_string(void);
size_t workspace_size(int B, int H, int Seq_q, int Seq_k);

#if defined(AAT_OP_ATTN)
/* Flash-attention forward.  Replaces: reference csrc/kernels/attention/regfuse/profile_code.py:30
 * (profile) and :68 (kernel_entry); csrc/kernels/attention/smemfuse/profile_code.py has the same pair.
 * Bound by reference python/autotuner/base_tunner.py:96-110 and python/autotuner/runtime.py:74-82. */
float profile(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k);
int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_k, int Seq_q);
float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q,
                 int Seq_k, float softmax_scale, int causal, void* workspace, size_t workspace_bytes,
                 void* stream);
int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q,
                    int Seq_k, float softmax_scale, int causal, void* workspace,
                    size_t workspace_bytes, void* stream);
/* kernel_entry_ex that also writes lse [B,H,Seq_q] fp32, the natural log-sum-exp of the scaled scores of
 * every query row (-inf for a row with no visible key), which the backward needs.  The reference computes
 * this value (csrc/kernels/attention/regfuse/regfuse.h:411) but never stores it and declares no such
 * entry point; its operator's commented-out `ctx.save_for_backward(q, k, v) # , lse)`
 * (python/ops/attention_interface.py:33) is the call site this serves. */
int kernel_entry_lse(aat_half* q, aat_half* k, aat_half* v, aat_half* o, float* lse, int B, int H,
                     int Seq_q, int Seq_k, float softmax_scale, int causal, void* workspace,
                     size_t workspace_bytes, void* stream);

#elif defined(AAT_OP_RET)
/* RetNet parallel forward.  Replaces: reference csrc/kernels/retnet/regfuse/profile_code.py:34 and :72
 * (and the smemfuse pair).  `causal` != 0 promises that mask is zero above the diagonal so those
 * tiles may be skipped. */
float profile(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B,
              int H, int Seq_q, int Seq_k);
int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B,
                 int H, int Seq_k, int Seq_q);
float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B,
                 int H, int Seq_q, int Seq_k, int causal, void* workspace, size_t workspace_bytes,
                 void* stream);
int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r,
                    int B, int H, int Seq_q, int Seq_k, int causal, void* workspace,
                    size_t workspace_bytes, void* stream);
/* The same with RetNet's decay mask built in registers instead of read from a tensor:
 * mask[h][i][j] = gamma_h^(i + Seq_k - Seq_q - j) for j <= i + Seq_k - Seq_q, 0 above that diagonal;
 * log2_gamma [H] fp32 holds log2(gamma_h), 0.5 <= gamma_h <= 1.  Tiles above the diagonal are skipped.
 * No counterpart in the reference, which always streams the [H,Seq_q,Seq_k] tensor
 * (python/ops/retnet_interface.py:26-31) and lists "causal config" and the mask stream's cost as open
 * items (README.md:102-114). */
float profile_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* o, float* r,
                    int B, int H, int Seq_q, int Seq_k, void* workspace, size_t workspace_bytes,
                    void* stream);
int kernel_entry_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* o,
                       float* r, int B, int H, int Seq_q, int Seq_k, void* workspace,
                       size_t workspace_bytes, void* stream);

#elif defined(AAT_OP_RET_BWD)
/* RetNet parallel backward.  Replaces: reference csrc/kernels/retnet/bwd/profile_code.py:53 and :98.
 * dqaccum is fp32 scratch the caller has zeroed; dq, dk, dv are fully overwritten.
 * A library built with a stored dS (configuration field ds_rows != 0) reports B*H*Seq_q*Seq_k fp16 more in
 * workspace_size(): given that room, the dQ pass writes the dS tiles it forms and dK comes from a kernel that
 * reads them back; given less (or none, as through the reference-signature entry points) dK comes from the
 * chained pass that evaluates dS a second time, with the results of a library built without it. */
float profile(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r,
              aat_half* dq, aat_half* dk, aat_half* dv, float* dqaccum, int B, int H, int Seq_q,
              int Seq_k);
int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r,
                 aat_half* dq, aat_half* dk, aat_half* dv, float* dqaccum, int B, int H, int Seq_k,
                 int Seq_q);
float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r,
                 aat_half* dq, aat_half* dk, aat_half* dv, float* dqaccum, int B, int H, int Seq_q,
                 int Seq_k, int causal, void* workspace, size_t workspace_bytes, void* stream);
int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r,
                    aat_half* dq, aat_half* dk, aat_half* dv, float* dqaccum, int B, int H, int Seq_q,
                    int Seq_k, int causal, void* workspace, size_t workspace_bytes, void* stream);
/* Decay-mask variant of the backward (see the forward's profile_decay); no dqaccum argument. */
float profile_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO, float* r,
                    aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k,
                    void* workspace, size_t workspace_bytes, void* stream);
int kernel_entry_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO,
                       float* r, aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q,
                       int Seq_k, void* workspace, size_t workspace_bytes, void* stream);

#elif defined(AAT_OP_ATTN_BWD)
/* Flash-attention backward: dq, dk, dv from q, k, v, o, dO and the forward's lse (see kernel_entry_lse).
 * No counterpart in the reference, whose MultiHeadAttnFunc.backward is an empty stub
 * (python/ops/attention_interface.py:37-58, README.md:107); this is the entry point that stub would bind.
 * Seq_q and Seq_k must both be multiples of the library's Br and Bc.  workspace_size() bytes of
 * workspace are required (two fp32 values per query row); dq, dk, dv are fully overwritten. */
float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, aat_half* dO, float* lse,
                 aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k,
                 float softmax_scale, int causal, void* workspace, size_t workspace_bytes, void* stream);
int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, aat_half* dO, float* lse,
                    aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k,
                    float softmax_scale, int causal, void* workspace, size_t workspace_bytes,
                    void* stream);

#elif defined(AAT_OP_RET_RECURRENT)
/* RetNet recurrent form, fp32:  S_n = decay[h][n] * S_{n-1} + k_n^T v_n,  out_n = q_n S_n  over the first
 * block_kdim key dims.  q, k [batch, heads, kdim, l], v, out [batch, heads, vdim, l] (sequence contiguous),
 * decay [heads, l]; every decay value is used as given (zero and negative ones included).
 * Replaces: reference csrc/kernels/retnet/recurrent/recurrent.h:427 (retnet_recurrent_fwd, same name and
 * arguments), whose only caller is benchmarks/retnet/retnet.cu:175-215.  This is ONE library for all
 * supported shapes: l a multiple of 32 (the reference reads whole 2048-position chunks, :453-460),
 * block_kdim a multiple of 64 up to 256 (the reference's MAX_KDIM, :18) and <= kdim, vdim a multiple of 64.
 * retnet_recurrent_workspace_size() bytes of workspace hold the per-(head, chunk) decay factors and, for
 * more than 128 key dims (contracted in passes of 128 whose outputs add), a second output-sized buffer;
 * workspace_size(B, H, l, l) is the same figure for up to 128 key dims.  The
 * reference-signature entry point has no workspace argument: up to 128 key dims and
 * AAT_RECURRENT_NOALLOC_MAX_RECORDS (head, chunk) pairs (the reference benchmark's shape among them) it keeps
 * the factors in the static array of retnet_recurrent_fwd_noalloc below and allocates nothing; beyond that it
 * is the one exception to "nothing is allocated by the callee" -- one buffer per device, grown on demand, kept
 * until the process ends.  It launches on the null stream and reports errors on stderr.  Every call on a
 * device uses that device's one array or buffer: calls that overlap on one GPU (other streams, other
 * threads) race; such callers take the _ex entry point with a workspace of their own. */
void retnet_recurrent_fwd(void* d_q, void* d_k, void* d_v, void* d_decay, void* d_out, int batch, int heads,
                          int kdim, int vdim, int l, int block_kdim);
size_t retnet_recurrent_workspace_size(int batch, int heads, int kdim, int vdim, int l, int block_kdim);
int retnet_recurrent_fwd_ex(const float* q, const float* k, const float* v, const float* decay, float* out,
                            int batch, int heads, int kdim, int vdim, int l, int block_kdim, void* workspace,
                            size_t workspace_bytes, void* stream);
float retnet_recurrent_profile(const float* q, const float* k, const float* v, const float* decay, float* out,
                               int batch, int heads, int kdim, int vdim, int l, int block_kdim, void* workspace,
                               size_t workspace_bytes, void* stream);
/* retnet_recurrent_fwd_ex without the workspace and without any allocation.  No counterpart in the
 * reference; it is for callers that cannot allocate device memory at the time of the call (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  The decay factors go into a
 * static device array inside the library, AAT_RECURRENT_NOALLOC_MAX_RECORDS records of 5120 bytes (15 MiB,
 * held by every GPU the library runs on until the process ends), so heads * (l / 32) must not exceed that
 * number and block_kdim must not exceed 128: AAT_ERR_LIMIT otherwise, AAT_ERR_SHAPE for what
 * retnet_recurrent_fwd_ex rejects too, 0 on success, a positive hipError_t from the runtime.  The first
 * call on a device looks the array's address up (hipGetSymbolAddress); make that call outside a capture.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU race. */
#define AAT_RECURRENT_NOALLOC_MAX_RECORDS 3072
int retnet_recurrent_fwd_noalloc(const float* q, const float* k, const float* v, const float* decay, float* out,
                                 int batch, int heads, int kdim, int vdim, int l, int block_kdim, void* stream);
#endif

#ifdef __cplusplus
}
#endif
#endif /* AAT_KERNEL_ABI_H */
