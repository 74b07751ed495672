/*
 * C ABI of libhbsattn_amd.so — hand-written gfx950 (MI355X) kernels for the
 * block-sparse attention forward that sits behind hbsattn.HBSAttention.
 *
 * The reference has no FFI for this path: its operator
 * (reference hbsattn/hbsa_interface.py:9-27) calls a Python launcher that JIT-compiles
 * a Triton kernel (reference hbsattn/fwd_triton_auto_tile_size.py:254-310 and
 * hbsattn/fwd_triton_fix_tile_size.py:216-276).  The entry points below are what a
 * binding for that launcher would need; each cites the reference code it replaces.
 *
 * Conventions
 *   - every pointer argument except `strides` / `mask_strides` (host arrays read during
 *     the call) is DEVICE memory owned by the caller; the library never allocates,
 *     frees or retains device memory;
 *   - all launches go to `stream` (a hipStream_t passed as void*; NULL = the null
 *     stream) and the calls return without synchronising;
 *   - return value 0 = success, negative = invalid argument (message available
 *     through hbsa_last_error(), which is thread-local), positive = hipError_t;
 *   - strides are in ELEMENTS; the innermost (head-dim) stride of q/k/v/out must be 1 and
 *     every row must start on a 16-byte boundary.  The token strides of k and v (and, in the
 *     backward, of q and dout) must lie in [0, 2^24]: the kernels address the
 *     rows of a tile with 32-bit offsets.  Other strides may take any value, negative included.
 */
#ifndef HBSATTN_AMD_H_
#define HBSATTN_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HBSA_ABI_VERSION 6

/* element types of q/k/v/out (reference: dtype follows the input tensors,
 * hbsattn/fwd_triton_auto_tile_size.py:272) */
#define HBSA_DTYPE_BF16 0
#define HBSA_DTYPE_F16 1
#define HBSA_DTYPE_F32 2          /* fp32 tensors, fp32 matrix instructions: the reference's fp32 arithmetic */
#define HBSA_DTYPE_F32_STAGED16 3 /* fp32 tensors, 16-bit matrix instructions: see hbsa_fwd_workspace_bytes_dtype */

#define HBSA_ERR_INVALID_ARGUMENT (-1)
#define HBSA_ERR_UNSUPPORTED (-2)
#define HBSA_ERR_WORKSPACE_TOO_SMALL (-3)

/* ABI version of the loaded library (== HBSA_ABI_VERSION it was built with). */
int hbsa_abi_version(void);

/* Message of the last failing call on this host thread ("" if none). */
const char *hbsa_last_error(void);

/*
 * Deterministic mode (process-wide; returns the previous setting).  It is ON by default: every query
 * block walks its kept key tiles in ascending order and results are bitwise reproducible at every size,
 * like the reference's kernels, which always scan in ascending order (reference
 * hbsattn/fwd_triton_auto_tile_size.py:153-164).  The attention kernel may visit the kept key tiles of
 * a query block in any order, and switching the mode OFF (hbsa_set_deterministic(0), or the environment
 * variable HBSATTN_AMD_DETERMINISTIC=0 when the library is loaded) lets very large problems use that:
 * when K and V of one kv head reach hbsa_set_walk_min_bytes (192 MiB unless changed; k_block_size a
 * multiple of 64) every query block's walk starts at the mean position of the workgroups that are
 * inside the same (kv head, sequence), kept in a clock word per (kv head, sequence) in the workspace,
 * and wraps around: those workgroups share an L2, and the K/V tiles one of them fetched are then found
 * there by the others (a seventh less HBM traffic and 5 % less time at 8 x 64K tokens, 30 % of the
 * blocks kept).  The fp32 summation order then depends on timing and results differ from run to run in
 * their last bits (the error against an exact evaluation is unchanged).
 */
int hbsa_set_deterministic(int on);

int hbsa_set_onepass(int on);   /* see hbsa_fwd */

/* Launches an hbsa_fwd call with these sizes would make on `stream` right now: 1 when its one-launch form
 * applies (the call then needs no workspace), else 2 (pre-pass and attention kernel; more for
 * HBSA_DTYPE_F32_STAGED16 and for work split over key blocks).  Host-side only, nothing is launched. */
int hbsa_fwd_launches(int32_t dtype, int32_t batch, int32_t total_k, int32_t nhead_q, int32_t nhead_k,
                      int32_t headdim, int32_t num_q_block, int32_t num_k_block,
                      int32_t q_block_size, int32_t k_block_size, int64_t mask_kblk_stride, void *stream);

/* Size (K + V bytes of one kv head) from which the clocked walk above is used; a negative value only
 * reads the setting.  Returns the previous value. */
long long hbsa_set_walk_min_bytes(long long bytes);

/*
 * Block geometry of a packed variable-length batch, on the HOST (all pointers are host memory):
 * the counterpart of hbsattn.utils.calculate_blocks (reference hbsattn/utils.py:7-50) for callers
 * without torch.  Blocks restart at every sequence start and the last block of a sequence may be
 * short.  Writes *num_block, cu_num_block[batch+1] (first global block of each sequence) and, when
 * given, cu_block[num_block+1] (token boundaries; cu_block[0] = 0 like the reference, which
 * assumes cu_seqlen[0] = 0) and block_to_batch[num_block]; `capacity` is the number of blocks the
 * last two can hold.  Call it with cu_block = block_to_batch = NULL to size them first.
 */
int hbsa_calculate_blocks(const int32_t *cu_seqlen, int32_t batch, int32_t block_size,
                          int32_t *num_block, int32_t *cu_num_block,
                          int32_t *cu_block, int32_t *block_to_batch, int32_t capacity);

/*
 * Bytes of device scratch hbsa_fwd needs for this problem.  Replaces the launcher's
 * own scratch allocations (reference hbsattn/fwd_triton_auto_tile_size.py:273-274:
 * `lse`, `tmp`); here the scratch holds the compacted work description the pre-pass
 * builds (per-q-block geometry records and one bit per in-sequence k block).
 * Depends only on host-known sizes, so no device synchronisation is needed.
 */
size_t hbsa_fwd_workspace_bytes(int32_t nhead_k, int32_t num_q_block, int32_t num_k_block);

/*
 * The same for a given element type.  For every type but HBSA_DTYPE_F32_STAGED16 it equals
 * hbsa_fwd_workspace_bytes.
 *
 * fp32 q/k/v/out (the reference accepts them, its tests use them: reference
 * test/test_accuracy.py:24) come in two forms.  HBSA_DTYPE_F32 multiplies fp32 operands with fp32
 * matrix instructions, as the reference's fp32 path does (tl.dot(..., allow_tf32=False), reference
 * hbsattn/fwd_triton_auto_tile_size.py:205,225), at the fp32 matrix rate, a sixteenth of the bf16
 * one.  HBSA_DTYPE_F32_STAGED16 is the fast form: each tensor is multiplied by a power of two
 * chosen from its largest magnitude (found on the device, no host synchronisation) and rounded to
 * fp16 staging copies in the workspace, the 16-bit kernel runs on those with fp32 accumulation and
 * softmax, and `out` is written as fp32.  Its operands carry 11-bit significands (fp32's range is
 * kept by the scaling): on unit-scale data the result differs from an all-fp32 evaluation by about
 * 1e-3 at most, inside the reference's own test tolerance (allclose with atol = rtol = 1e-2,
 * reference test/test_accuracy.py:87-89).
 * hbsa_fwd_prepare needs only the hbsa_fwd_workspace_bytes prefix.
 */
size_t hbsa_fwd_workspace_bytes_dtype(int32_t dtype, int32_t total_q, int32_t total_k,
                                      int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                                      int32_t num_q_block, int32_t num_k_block);

/*
 * Extra bytes, behind the hbsa_fwd_workspace_bytes_dtype(...) bytes of the same workspace, that let
 * hbsa_fwd / hbsa_fwd_run split the work over key blocks when there are too few (kv head, q block)
 * work items to fill the current device (short query side, long key side): every item is cut
 * into up to 32 parts over its k blocks, the parts run as separate work items and a merge kernel
 * combines their normalised partial results through their log-sum-exps.  0 when the split would
 * not be used for this shape on this device.  A workspace without these bytes is valid; the call
 * then runs unsplit.  The reference has no counterpart (one program per q tile,
 * reference hbsattn/fwd_triton_auto_tile_size.py:283).
 */
size_t hbsa_fwd_split_workspace_bytes(int32_t total_q, int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                                      int32_t num_q_block, int32_t num_k_block, int32_t q_block_size);

/*
 * Block-sparse attention forward.  Replaces `_forward_auto_tile_size` and
 * `_forward_fix_tile_size` + their Triton `_fwd_kernel`s (reference
 * hbsattn/fwd_triton_auto_tile_size.py:76-310, hbsattn/fwd_triton_fix_tile_size.py:30-276).
 *
 *   q   [total_q, nhead_q, headdim]   k, v [total_k, nhead_k, headdim]   out like q
 *   cu_q_seqlens, cu_k_seqlens  int32[batch+1]  packed-sequence boundaries
 *   block_mask  bytes (0 / non-0) [nhead_k, num_q_block, num_k_block] over GLOBAL block
 *               indices; entries pairing blocks of different sequences are ignored
 *   q_block_to_batch int32[num_q_block], cu_num_q_block / cu_num_k_block int32[batch+1]
 *               exactly as hbsattn.utils.calculate_blocks returns them
 *               (reference hbsattn/utils.py:7-50)
 *   causal      bottom-right aligned: in-sequence key j visible to in-sequence query i
 *               iff i + (k_len - q_len) >= j
 *   softmax_scale  already resolved (the caller substitutes headdim**-0.5 for None)
 *   strides     int64[11] = { q_tok, q_head, k_tok, k_head, v_tok, v_head,
 *                             out_tok, out_head, mask_head, mask_qblk, mask_kblk }
 *   workspace   >= hbsa_fwd_workspace_bytes_dtype(...) bytes, 256-byte aligned; may be NULL (with
 *               workspace_bytes 0) for a call that runs as one launch, see below
 *
 * Launches.  In general the call is two launches, hbsa_fwd_prepare's pre-pass (mask bytes and sequence
 * boundaries -> a compact work description in `workspace`) and the attention kernel.  A call on bf16 or
 * fp16 tensors is ONE launch, and does not touch `workspace`, when the attention kernel's scheduler can
 * read the boundaries and the mask bytes itself: mask_kblk stride 1, at most 127 sequences, work that
 * would neither be split over key blocks (hbsa_fwd_split_workspace_bytes) nor use the clocked walk,
 * `stream` not being captured into a graph, and fewer than 64 other streams of the device having made such
 * calls.  The launch record (work-queue counters) of that form lives in device memory inside the library,
 * one record per stream, so calls on different streams may overlap; it replaces the reference kernel's
 * per-program scan of the mask (reference hbsattn/fwd_triton_auto_tile_size.py:153-164) and the
 * launcher's two host synchronisations (:276-277) with nothing at all.  Results are bitwise those of the
 * two-launch path.  A call that cannot run as one launch and has no (or too small a) workspace returns
 * HBSA_ERR_WORKSPACE_TOO_SMALL before anything is launched.  hbsa_set_onepass(0) switches the form off
 * (process-wide; returns the previous setting; the environment variable HBSATTN_AMD_ONEPASS=0 does the same
 * when the library is loaded).
 *
 * Supported: headdim in {32, 64, 128, 256} (the reference pads any head dim to the next power of two,
 * reference hbsattn/fwd_triton_auto_tile_size.py:269; callers do the same with zero columns up to one of
 * these); q_block_size, k_block_size positive multiples of 16; nhead_q % nhead_k == 0; every sequence
 * length >= 1.  At headdim 256 a CU runs one workgroup of four wavefronts whose operand reads the compiler
 * schedules: it works, at about two thirds of the efficiency of headdim 128.  Query rows with no
 * visible key produce exactly 0 (reference hbsattn/reference.py:97-98).
 */
int hbsa_fwd(const void *q, const void *k, const void *v, void *out,
             const int32_t *cu_q_seqlens, const int32_t *cu_k_seqlens,
             const uint8_t *block_mask,
             const int32_t *q_block_to_batch, const int32_t *cu_num_q_block,
             const int32_t *cu_num_k_block,
             void *workspace, size_t workspace_bytes,
             int32_t dtype, int32_t batch, int32_t total_q, int32_t total_k,
             int32_t nhead_q, int32_t nhead_k, int32_t headdim,
             int32_t num_q_block, int32_t num_k_block,
             int32_t q_block_size, int32_t k_block_size,
             int32_t causal, float softmax_scale,
             const int64_t *strides, void *stream);

/*
 * hbsa_fwd with its arguments in arrays, for bindings that pay per argument (Python's ctypes spends more
 * host time on hbsa_fwd's 27 arguments than a small problem's kernel runs).  Same checks, launches and
 * results as hbsa_fwd:
 *   ptrs   host array of 11 pointers = { q, k, v, out, cu_q_seqlens, cu_k_seqlens, block_mask,
 *          q_block_to_batch, cu_num_q_block, cu_num_k_block, workspace }
 *   sizes  host array of 12 ints = { dtype, batch, total_q, total_k, nhead_q, nhead_k, headdim,
 *          num_q_block, num_k_block, q_block_size, k_block_size, causal }
 * Both arrays are read during the call only.
 */
int hbsa_fwd_v(const void *const *ptrs, size_t workspace_bytes, const int32_t *sizes, float softmax_scale,
               const int64_t *strides, void *stream);

/*
 * hbsa_fwd for callers that cannot allocate device memory or pass a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose launcher allocates its scratch with torch on every call, reference
 * hbsattn/fwd_triton_auto_tile_size.py:273-274).  Same arguments and results as hbsa_fwd without
 * `workspace` / `workspace_bytes`: the work description lives in a device array of
 * HBSA_STATIC_SCRATCH_BYTES inside the library, which every GPU the library runs on holds until the
 * process ends.  The call allocates and frees nothing.  A problem whose
 * hbsa_fwd_workspace_bytes_dtype(...) exceeds HBSA_STATIC_SCRATCH_BYTES is refused with
 * HBSA_ERR_WORKSPACE_TOO_SMALL before anything is launched.  All calls on one GPU share that GPU's
 * array: calls on one stream are ordered and safe; calls that overlap on one GPU (different streams
 * or host threads) race on it and must be serialised by the caller.  The first call on a device looks
 * up the array's address and the kernels' launch limits (host-side queries, no allocation): make it
 * before a stream capture begins, not inside one.  The call always runs as pre-pass + attention kernel on
 * the array (never as hbsa_fwd's one-launch form, whose launch record belongs to a stream), so it can be
 * recorded into a graph and the graph replayed on any stream.
 */
#define HBSA_STATIC_SCRATCH_BYTES (32u << 20)
int hbsa_fwd_static(const void *q, const void *k, const void *v, void *out,
                    const int32_t *cu_q_seqlens, const int32_t *cu_k_seqlens,
                    const uint8_t *block_mask,
                    const int32_t *q_block_to_batch, const int32_t *cu_num_q_block,
                    const int32_t *cu_num_k_block,
                    int32_t dtype, int32_t batch, int32_t total_q, int32_t total_k,
                    int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                    int32_t num_q_block, int32_t num_k_block,
                    int32_t q_block_size, int32_t k_block_size,
                    int32_t causal, float softmax_scale,
                    const int64_t *strides, void *stream);

/*
 * The two halves of hbsa_fwd, for callers that apply one block mask to many q/k/v
 * (layers or steps sharing a sparsity pattern) or that time the kernels separately.
 *
 * hbsa_fwd_prepare runs the pre-pass only: it turns block_mask + sequence boundaries into
 * the compact work description inside `workspace`.  It replaces the per-program mask scan
 * of the reference kernel (reference hbsattn/fwd_triton_auto_tile_size.py:153-164: every
 * program loads one mask byte per k block of its sequence and branches on it).
 *   mask_strides  int64[3] = { mask_head, mask_qblk, mask_kblk } in elements (bytes)
 *   total_q, total_k  token rows of the q and k/v tensors the workspace will be run with.  The sequence
 *                 boundaries are device data the host cannot check; the pre-pass checks them against
 *                 these bounds and the block counts, and a sequence that does not fit (q/k/v shorter than
 *                 cu_seqlens says, inconsistent block metadata) gets no keys: nothing of k, v or the mask is
 *                 read for it, and those of its query rows that lie inside q get zeros in `out` (and zero
 *                 gradients in the backward), like any row that sees no key.  The reference reads and
 *                 writes out of bounds in that case.
 *
 * hbsa_fwd_run runs the attention kernel from a prepared `workspace` (same sizes, block
 * sizes and `causal` as the prepare call; q/k/v/out and softmax_scale may differ per call).
 * It advances the work-queue counters inside `workspace` (hbsa_fwd_prepare leaves them at zero and
 * every attention launch puts them back to zero as its last workgroup ends, so a prepared workspace
 * can be run any number of times with no step in between); two runs that share one workspace must
 * therefore be ordered on one stream, not concurrent.
 * It replaces the reference `_fwd_kernel` launch (reference
 * hbsattn/fwd_triton_auto_tile_size.py:283-308).
 *   strides       int64[8] = { q_tok, q_head, k_tok, k_head, v_tok, v_head, out_tok, out_head }
 */
int hbsa_fwd_prepare(const int32_t *cu_q_seqlens, const int32_t *cu_k_seqlens,
                     const uint8_t *block_mask,
                     const int32_t *q_block_to_batch, const int32_t *cu_num_q_block,
                     const int32_t *cu_num_k_block,
                     void *workspace, size_t workspace_bytes,
                     int32_t batch, int32_t nhead_k, int32_t num_q_block, int32_t num_k_block,
                     int32_t q_block_size, int32_t k_block_size, int32_t causal,
                     int32_t total_q, int32_t total_k,
                     const int64_t *mask_strides, void *stream);

int hbsa_fwd_run(const void *q, const void *k, const void *v, void *out,
                 void *workspace, size_t workspace_bytes,
                 int32_t dtype, int32_t total_q, int32_t total_k,
                 int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                 int32_t num_q_block, int32_t num_k_block,
                 int32_t q_block_size, int32_t k_block_size,
                 int32_t causal, float softmax_scale,
                 const int64_t *strides, void *stream);

/*
 * hbsa_fwd_run that also writes, per query row and q head, the natural logarithm of the sum over
 * the row's visible keys of exp(softmax_scale * q.k) (-inf for a row without visible keys):
 * what merging attention over disjoint key sets needs.  The reference computes a per-row
 * `lse` scratch but without the running maximum and does not return it
 * (reference hbsattn/fwd_triton_auto_tile_size.py:246-251, 273, 310); this is the complete value.
 *   lse           float [total_q, nhead_q] with element strides lse_strides = { tok, head };
 *                 NULL = same as hbsa_fwd_run
 */
int hbsa_fwd_run_lse(const void *q, const void *k, const void *v, void *out,
                     float *lse, const int64_t *lse_strides,
                     void *workspace, size_t workspace_bytes,
                     int32_t dtype, int32_t total_q, int32_t total_k,
                     int32_t nhead_q, int32_t nhead_k, int32_t headdim,
                     int32_t num_q_block, int32_t num_k_block,
                     int32_t q_block_size, int32_t k_block_size,
                     int32_t causal, float softmax_scale,
                     const int64_t *strides, void *stream);

/*
 * Backward of the block-sparse attention forward: dq, dk, dv from dout = d loss / d out.
 * The reference has no counterpart: its operator's backward raises NotImplementedError
 * (reference hbsattn/hbsa_interface.py:31-32); the gradients are those of the forward the reference
 * defines (reference hbsattn/reference.py:23-107).
 *
 *   q, out, dout, dq [total_q, nhead_q, headdim]     k, v, dk, dv [total_k, nhead_k, headdim]
 *   lse         float [total_q, nhead_q], contiguous: what hbsa_fwd_run_lse wrote for the same
 *               q/k/v, mask and softmax_scale
 *   workspace   as left by hbsa_fwd_prepare (or hbsa_fwd) for the same mask, sequence boundaries,
 *               block sizes and `causal`; read only
 *   bwd_workspace  >= hbsa_bwd_workspace_bytes(total_q, nhead_q) bytes of device scratch, 16-byte aligned
 *               (two floats per (row, q head): rowsum(dout * out) and the scaled log-sum-exp)
 *   strides     int64[16] = { q_tok, q_head, k_tok, k_head, v_tok, v_head, out_tok, out_head,
 *                             dout_tok, dout_head, dq_tok, dq_head, dk_tok, dk_head, dv_tok, dv_head }
 *
 * Supported: HBSA_DTYPE_BF16 and HBSA_DTYPE_F16, headdim in {32, 64, 128}.  Every element of dq, dk
 * and dv is written (zeros where no gradient flows); no atomics, so results are deterministic.
 * There are no fp32 backward kernels: the fp32 matrix rate is a sixteenth of the 16-bit one and a backward
 * is 2.5 forwards of matrix work.  A caller with fp32 tensors passes bf16 copies of q, k, v, out and dout
 * (bf16 keeps fp32's range), with out and lse from a forward on those copies, and widens the gradients, which
 * is what the Python operator does.
 * Head dims above 128 are refused: the dK/dV kernel keeps K^T or V^T of a wavefront's keys and one accumulator
 * in registers, 254 of 256 at headdim 128.
 */
size_t hbsa_bwd_workspace_bytes(int32_t total_q, int32_t nhead_q);

int hbsa_bwd(const void *q, const void *k, const void *v, const void *out, const void *dout,
             const float *lse, void *dq, void *dk, void *dv,
             const int32_t *cu_k_seqlens, const int32_t *cu_num_q_block, const int32_t *cu_num_k_block,
             const void *workspace, size_t workspace_bytes,
             void *bwd_workspace, size_t bwd_workspace_bytes,
             int32_t dtype, int32_t batch, int32_t total_q, int32_t total_k,
             int32_t nhead_q, int32_t nhead_k, int32_t headdim,
             int32_t num_q_block, int32_t num_k_block,
             int32_t q_block_size, int32_t k_block_size,
             int32_t causal, float softmax_scale,
             const int64_t *strides, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HBSATTN_AMD_H_ */
