/*
 * mercury_hip.h -- C ABI of the MI355X (gfx950) ring-attention step library.
 *
 * One shared library, libmercury_hip.so, plain pointers and sizes only.  Every pointer
 * is a DEVICE pointer unless stated otherwise; `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  All calls are asynchronous on `stream`, allocate
 * nothing and keep no global mutable state (mhip_attn_bwd_block_noalloc excepted: it owns
 * a scratch array on every GPU).  Return value: 0 on success, a negative
 * MHIP_E* code otherwise (mhip_error_string() gives the text).  Nothing throws.
 *
 * Tensor layouts follow the call sites of the reference (paths relative to the
 * reference tree):
 *   q, out, dout, dq      (B, Sq, Hq,  D)   element strides (sb, ss, sh), D contiguous
 *   k, v, dk, dv          (B, Sc, Hkv, D)   element strides (sb, ss, sh), D contiguous
 *   lse (block / final)   (B, Hq, Sq)  fp32 contiguous
 *   merge accumulators    out (B, Sq, Hq, D) fp32, lse (B, Sq, Hq, 1) fp32, row strides given
 *   packed reduce buffer  (B, Sq, Hq, D+1) fp32, out in [0,D), lse in column D
 */
#ifndef MERCURY_HIP_H_
#define MERCURY_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes --------------------------------------------------------------- */
#define MHIP_OK              0
#define MHIP_EINVAL         -1   /* bad size / NULL pointer / bad scale                 */
#define MHIP_EDTYPE         -2   /* dtype code not supported by this entry point       */
#define MHIP_EHEADDIM       -3   /* head dimension not supported (see the entry point)  */
#define MHIP_EALIGN         -4   /* pointer or stride not 16-byte aligned              */
#define MHIP_ELAUNCH        -5   /* hipLaunchKernel / hipGetLastError reported failure */
#define MHIP_EUNSUPPORTED   -6   /* feature not implemented (dropout, alibi, window..) */
#define MHIP_ETOOLARGE      -7   /* problem exceeds the built-in scratch of a *_noalloc entry point */
#define MHIP_ERUNTIME       -8   /* a HIP runtime query (device, symbol address) failed */

/* ---- element types -------------------------------------------------------------- */
#define MHIP_BF16  0
#define MHIP_E4M3  1   /* OCP float8 e4m3fn */
#define MHIP_F32   2   /* input type of mhip_quantize_e4m3 only */

/* ---- mask classes of one (Q shard, KV chunk) block -------------------------------- */
#define MHIP_MASK_NONE    0
#define MHIP_MASK_CAUSAL  1   /* query i sees key j iff j <= i + (Sc - Sq) (bottom-right) */

/* Bumped whenever an entry point's argument list changes (a caller built against another value must not call).
 * 3: the three descales of mhip_attn_fwd_block are device pointers; mhip_attn_bwd_block takes five stride triples. */
#define MHIP_ABI_VERSION 3
int         mhip_abi_version(void);   /* the MHIP_ABI_VERSION the library was built with */
int         mhip_version(void);
/* Optional: per-device set-up the entry points otherwise do on their first call on a device (today: the address
 * of the scratch of mhip_attn_bwd_block_noalloc).  Cheap, idempotent, allocates nothing; MHIP_ERUNTIME if the
 * runtime query fails.  Call it outside stream capture. */
int         mhip_init(void);
const char* mhip_error_string(int code);

/*
 * Block forward: out = softmax(scale * q k^T) v,  lse = logsumexp(scale * q k^T).
 * Replaces flash_attn.flash_attn_interface._flash_attn_forward as called at
 * utils/flash_attn_dsl.py:159-176 (dropout_p = 0, softcap = 0, no alibi, window (-1,-1)).
 * out has q's element type for MHIP_BF16 and is bf16 for MHIP_E4M3.  Rows that see no key
 * get out = 0 and lse = -inf.  For MHIP_E4M3 the three descales point to the per-tensor fp32
 * scales s (x ~ s * x_q) in DEVICE memory, one float each, read by the kernel when it runs (so
 * they may be written by earlier work on the stream, and a captured graph uses the values present
 * at replay); NULL means 1.  They must be positive and finite (not checked: the values never
 * reach the host).  Ignored for MHIP_BF16.
 * Head dimension: MHIP_BF16 any multiple of 8 up to 128 (the kernel computes on 128 columns, on 64 for D <= 64;
 * the missing ones are zeros that exist only on chip -- no padded copy, no extra memory traffic -- and the K / V
 * span Sc * stride of one (batch, head) must stay below 2^30 bytes, MHIP_EUNSUPPORTED beyond); MHIP_E4M3 any
 * multiple of 16 up to 128, in the same way.  MHIP_EHEADDIM otherwise.
 */
int mhip_attn_fwd_block(const void* q, const void* k, const void* v, void* out, float* lse,
                        int B, int Sq, int Sc, int Hq, int Hkv, int D,
                        int64_t q_sb, int64_t q_ss, int64_t q_sh,
                        int64_t k_sb, int64_t k_ss, int64_t k_sh,
                        int64_t v_sb, int64_t v_ss, int64_t v_sh,
                        int64_t o_sb, int64_t o_ss, int64_t o_sh,
                        float softmax_scale, int mask, int dtype,
                        const float* q_descale, const float* k_descale, const float* v_descale,
                        void* stream);

/*
 * Block backward from the saved (final, merged) out and lse.
 * Replaces flash_attn.flash_attn_interface._flash_attn_backward as called at
 * utils/attn_bwd_dsl.py:83-115: writes every element of dq (B,Sq,Hq,D), dk and dv
 * (B,Sc,Hkv,D) in bf16.  If dq_acc (fp32, contiguous (B,Sq,Hq,D)) is not NULL the block's
 * dq is ALSO added into it in fp32 -- the `reduce(op=torch.add, buffer=reduce_dq, ...)`
 * of utils/attn_bwd_dsl.py:117-122 folded into the kernel.  `workspace` must hold
 * mhip_attn_bwd_workspace_bytes(...) bytes of device memory: three (B, Hq, Sq) fp32 arrays, each rounded up to a
 * multiple of 4 elements -- -delta (= -rowsum(dout * out), stored negated because the kernels start dP from it),
 * the LSE in base 2, and delta itself, which is what flash-attn returns as softmax_d.  dq and out have element strides of their own:
 * the call site allocates block_dq with torch.empty (contiguous, utils/attn_bwd_dsl.py:83) while q, out and
 * dout are views of the step's buffers; q and dout, k and v, dk and dv share a stride triple each.
 * Head dimension: any multiple of 8 up to 128, as for the bf16 forward (for D < 128 the q / dout span of one
 * batch and the k / v span of one (batch, head) must stay below 2^30 bytes).
 */
int64_t mhip_attn_bwd_workspace_bytes(int B, int Sq, int Sc, int Hq, int Hkv, int D);
int mhip_attn_bwd_block(const void* dout, const void* q, const void* k, const void* v,
                        const void* out, const float* lse,
                        void* dq, void* dk, void* dv, float* dq_acc,
                        int B, int Sq, int Sc, int Hq, int Hkv, int D,
                        int64_t q_sb, int64_t q_ss, int64_t q_sh,     /* q, dout  */
                        int64_t k_sb, int64_t k_ss, int64_t k_sh,     /* k, v     */
                        int64_t dk_sb, int64_t dk_ss, int64_t dk_sh,  /* dk, dv   */
                        int64_t dq_sb, int64_t dq_ss, int64_t dq_sh,  /* dq       */
                        int64_t o_sb, int64_t o_ss, int64_t o_sh,     /* out      */
                        float softmax_scale, int mask, int deterministic,
                        void* workspace, void* stream);

/*
 * mhip_attn_bwd_block without the workspace argument.  No counterpart in the reference: it is for callers
 * that cannot hand over (or allocate) scratch memory -- code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc.  delta and lse2 go to an array built into the library (a file-scope
 * __device__ array of 8 MiB + 32 bytes, held by every GPU the library runs on until the process ends), so
 * the block is limited to B * Hq * Sq <= 1048576 (MHIP_ETOOLARGE beyond).  The first call on a device asks
 * the runtime for that device's address of the array (hipGetSymbolAddress, MHIP_ERUNTIME if that fails), which
 * is a runtime query and must not happen while the stream is being captured: call mhip_init() on the device
 * first (or make one eager call) before recording this entry point into a HIP graph.
 * No call allocates or frees.  All calls on one GPU share the array: calls that overlap in time on one GPU
 * (different streams, different threads) race on it and must be serialised by the caller.  Arguments,
 * results and error codes are otherwise those of mhip_attn_bwd_block.
 */
int mhip_attn_bwd_block_noalloc(const void* dout, const void* q, const void* k, const void* v,
                                const void* out, const float* lse,
                                void* dq, void* dk, void* dv, float* dq_acc,
                                int B, int Sq, int Sc, int Hq, int Hkv, int D,
                                int64_t q_sb, int64_t q_ss, int64_t q_sh,     /* q, dout  */
                                int64_t k_sb, int64_t k_ss, int64_t k_sh,     /* k, v     */
                                int64_t dk_sb, int64_t dk_ss, int64_t dk_sh,  /* dk, dv   */
                                int64_t dq_sb, int64_t dq_ss, int64_t dq_sh,  /* dq       */
                                int64_t o_sb, int64_t o_ss, int64_t o_sh,     /* out      */
                                float softmax_scale, int mask, int deterministic, void* stream);

/*
 * LSE-rescale merge.  Replaces the TorchScript `_update_out_and_lse`
 * (utils/flash_attn_dsl.py:31-49):
 *     out' = out - sigmoid(bl - lse) * (out - bo),   lse' = lse - logsigmoid(lse - bl)
 * with bo = float(block_out), bl = block_lse read transposed from (B,Hq,Sq).
 * acc_out/acc_lse are read, dst_out/dst_lse written; dst may alias acc (the `slice_`
 * path of utils/flash_attn_dsl.py:63-68 passes views, hence the strides: element strides
 * of the (B,Sq,Hq) row index; D is contiguous).  A -inf operand is the identity.
 * acc_out == NULL means "first call" (utils/flash_attn_dsl.py:61-62): dst = (bo, bl).
 * If final_out / final_lse are not NULL the epilogue of utils/flash_attn_dsl.py:178-179 is
 * fused: final_out (B,Sq,Hq,D) bf16 contiguous = bf16(out'), final_lse (B,Hq,Sq) = lse'.
 * block_lse rows are addressed as block_lse[b*bl_sb + h*bl_sh + s].
 */
int mhip_lse_merge(const float* acc_out, const float* acc_lse,
                   const void* block_out, const float* block_lse,
                   float* dst_out, float* dst_lse,
                   void* final_out, float* final_lse,
                   int B, int Sq, int Hq, int D,
                   int64_t ao_sb, int64_t ao_ss, int64_t ao_sh,
                   int64_t al_sb, int64_t al_ss, int64_t al_sh,
                   int64_t bo_sb, int64_t bo_ss, int64_t bo_sh,
                   int64_t bl_sb, int64_t bl_sh,
                   int64_t do_sb, int64_t do_ss, int64_t do_sh,
                   int64_t dl_sb, int64_t dl_ss, int64_t dl_sh,
                   void* stream);

/*
 * All block results of a ring step folded at once.  Replaces the chain of N update_out_and_lse calls of
 * the chunk loop (utils/flash_attn_dsl.py:51-71, one per chunk) together with the stores of
 * utils/flash_attn_dsl.py:178-179: with L = logsumexp_i(lse_i),
 *   final_out = bf16(sum_i exp(lse_i - L) * out_i),  final_lse = L,
 * which is what the chain computes (the fold is associative) without moving the fp32 accumulator through
 * memory N - 1 times.  block_outs / block_lses / bo_sb / s_begin are HOST arrays of n entries
 * (1 <= n <= 64; s_begin may be NULL = all zero).  Block i covers the sequence rows s >= s_begin[i]
 * (rows before count as lse = -inf: the "second half of the Q rows" steps of a zigzag schedule):
 * block_outs[i] bf16 (B, Sq - s_begin[i], Hq, D) addressed with the element strides bo_sb[i], bo_ss, bo_sh
 * (multiples of 8, 16-byte aligned base, D contiguous), block_lses[i] fp32 (B, Hq, Sq - s_begin[i])
 * contiguous.  final_out bf16 (B,Sq,Hq,D) contiguous, final_lse fp32 (B,Hq,Sq) contiguous.
 * D a multiple of 8 up to 256.  Rows whose lse is -inf in every block get (0, -inf).
 */
int mhip_lse_merge_many(const void* const* block_outs, const float* const* block_lses,
                        const int64_t* bo_sb, const int* s_begin, int n,
                        void* final_out, float* final_lse,
                        int B, int Sq, int Hq, int D,
                        int64_t bo_ss, int64_t bo_sh, void* stream);

/*
 * Packed merge.  Replaces TorchScript `flash_reduce` (utils/flash_attn_dsl.py:293-305):
 * lhs, rhs, dst are contiguous fp32 (rows, D+1), 16-byte aligned; dst must not overlap lhs
 * or rhs (MHIP_EINVAL; the reference's flash_reduce returns a new tensor as well).
 */
int mhip_flash_reduce(const float* lhs, const float* rhs, float* dst,
                      int64_t rows, int D, void* stream);

/* Tree-attention merge of packed (rows, D+1) fp32 operands (out | lse) across ranks: replaces the local
 * arithmetic of update_out_and_lse_collective, utils/flash_attn_dsl.py:307-324 (the collectives stay with
 * the caller).  With row_max[r] = max over ranks of the lse column (one MAX all-reduce of `rows` floats):
 *   finish == 0:  dst = (out * d | d), d = exp(lse - row_max)   -- this rank's term of ONE SUM all-reduce
 *   finish != 0:  src is the summed terms; dst = (sum_out / sum_d | row_max + log(sum_d))
 * dst may be src itself (in place; any other overlap of the two is rejected with MHIP_EINVAL).  Rows with
 * row_max = -inf come out as (0 | -inf). */
int mhip_tree_merge(const float* src, const float* row_max, float* dst, int64_t rows, int D, int finish,
                    void* stream);

/*
 * Per-tensor e4m3 quantisation for the fp8 forward path (not in the reference, whose ring templates run
 * bf16 only; the block kernel's descales are the scales this writes): scale = amax(|x|) / 448 (1 when the
 * tensor is all zero), xq = round-to-nearest-even e4m3fn(clamp(x / scale, -448, 448)), bit for bit what
 * (x.float() / scale).clamp(-448, 448).to(torch.float8_e4m3fn) gives.  x: n contiguous elements of
 * MHIP_F32 or MHIP_BF16, 16-byte aligned; xq: n bytes, 8-byte aligned; scale: one fp32 on the device;
 * amax_ws: 4 bytes of device scratch.  Three launches on the stream.
 */
int mhip_quantize_e4m3(const void* x, int dtype, int64_t n, void* xq, float* scale, float* amax_ws,
                       void* stream);

/*
 * Pack a block result: dst (B,Sq,Hq,D+1) fp32 contiguous =
 * cat([float(block_out), block_lse^T], -1)   (utils/flash_attn_dsl.py:396).
 * If lhs is not NULL the pack is fused with the reduce: dst = flash_reduce(lhs, pack(block));
 * dst must not overlap lhs (MHIP_EINVAL); dst and lhs 16-byte aligned.  block_out (B,Sq,Hq,D) bf16 and block_lse
 * (B,Hq,Sq) contiguous.
 */
int mhip_pack_reduce(const float* lhs, const void* block_out, const float* block_lse,
                     float* dst, int B, int Sq, int Hq, int D, void* stream);

/*
 * Epilogue of the packed form.  Replaces `o[...] = buf[..., :-1].to(q.dtype)` and
 * `lse[...] = buf[..., -1].transpose(1, 2)` (the stores after the managed reduction,
 * utils/flash_attn_dsl.py:406-407): buf fp32 (B,Sq,Hq,D+1) contiguous, out bf16 (B,Sq,Hq,D)
 * contiguous and 16-byte aligned, lse fp32 (B,Hq,Sq) contiguous.  D a multiple of 8 that divides 2048.
 */
int mhip_unpack(const float* buf, void* out, float* lse, int B, int Sq, int Hq, int D, void* stream);

/*
 * Gradient accumulation `torch.add(buf, block.to(float32))` (utils/attn_bwd_dsl.py:117-129):
 * dst = (acc ? acc : 0) + float(block), n elements, block in bf16; dst may alias acc.
 */
int mhip_grad_accumulate(const float* acc, const void* block, float* dst, int64_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MERCURY_HIP_H_ */
