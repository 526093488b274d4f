/*
 * varq.h -- C ABI of libvarq_hip.so: VAR-Q KV-cache quantization hot path for
 * AMD MI355X (gfx950).
 *
 * The reference (lujiaji/VAR-Q) is pure Python and has no FFI; the interface
 * replaced here is its Python surface.  Each entry point cites the reference
 * lines whose work it performs.  Conventions common to every call:
 *
 *   - all pointers are DEVICE pointers unless named host_*; the library never
 *     allocates, frees, synchronizes or keeps a pointer after returning;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - return value 0 = success, negative = one of varq_status; the message for
 *     the calling thread's last failure is varq_last_error();
 *   - shapes are validated on the host before any launch; nothing is launched
 *     when validation fails;
 *   - dtype codes: 0 = fp32, 1 = bf16, 2 = fp16;
 *   - codes are signed two's complement in [-(2^(b-1)), 2^(b-1)-1]; packed
 *     words hold 32/bits codes, code j of a word at bit j*bits, along the last
 *     dimension (VAR_Q/pack_unpack.py:177-196).
 */
#ifndef VARQ_H
#define VARQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VARQ_ABI_VERSION 8

enum varq_status {
  VARQ_OK = 0,
  VARQ_ERR_INVALID = -1,     /* bad argument (shape, bits, dtype, null pointer) */
  VARQ_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for      */
  VARQ_ERR_LAUNCH = -3,      /* HIP reported an error at launch                 */
  VARQ_ERR_WORKSPACE = -4    /* workspace too small                             */
};

enum varq_dtype { VARQ_F32 = 0, VARQ_BF16 = 1, VARQ_F16 = 2 };

/* K/V tensor layouts of the reference's quantizer (qkv_format, VAR_Q/quant.py:34-37) */
enum varq_layout { VARQ_LAYOUT_BHLC = 0, VARQ_LAYOUT_BLHC = 1,
                   /* attention calls only: q and the cache as VARQ_LAYOUT_BHLC, out as VARQ_LAYOUT_BLHC */
                   VARQ_LAYOUT_BHLC_OUT_BLHC = 2 };

/*
 * What the matrix operands of the fused attention hold.
 * VARQ_ATTN_REFERENCE_ROUNDING (the default form): K and V are dequantized as tiles enter LDS,
 *   (code - zp) * scale in fp32, and rounded to the attention's 16-bit type -- the very operands
 *   the reference's attention backend sees after dequant_all() and the downcast of its call
 *   (VAR_Q/quant.py:216-224, VAR/models/basic_var.py:158, Infinity/infinity/models/basic.py:344).
 * VARQ_ATTN_EXACT_CODES (opt-in): the operands are exact images of the integer codes, scales
 *   and zero-points are applied in fp32 to the products, so K and V are never rounded.  Closer
 *   to the unrounded mathematics than the reference itself (whose bf16 rounding of K and V
 *   moves an output by up to a few percent of its range on heavy-tailed data), hence farther
 *   from the reference; a few percent faster.  Exists for one scale group per key of 4- or
 *   2-bit codes at D = 128 in bf16; every other shape computes with reference rounding whatever
 *   is asked for.
 */
enum varq_attn_form { VARQ_ATTN_REFERENCE_ROUNDING = 0, VARQ_ATTN_EXACT_CODES = 1 };

int varq_abi_version(void);
const char *varq_last_error(void);

/*
 * Row mapping used by the calls that write into a pre-allocated packed cache.
 * The input is seen as [n0, n1, n2] rows of `c` channels (the three leading
 * dims of the 4-D K/V tensor).  Row (i0,i1,i2) is written to output row
 *     s(i0,0)*os0 + s(i1,1)*os1 + s(i2,2)*os2 + off
 * where s(i,d) = slot[i] if d == slot_dim (rows whose slot is negative are
 * skipped) and i otherwise.  This is how a [B,H,n,c] step lands at token
 * offset L0 of a [B,H',Lmax,...] cache, optionally only the heads of one
 * bit-width class.  It replaces the torch.cat growth of VAR_Q/quant.py:200-201.
 * Passed as 8 host int64: {n0,n1,n2,os0,os1,os2,off,slot_dim(-1 = none)}.
 * A token-major step [B,n,H,c] goes into the same cache with the map
 * {B,n,H, H'*Lmax,1,Lmax, L0, 2}: the quantizer walks whichever of the inner two
 * dims has output stride 1, so both orders store whole contiguous stretches.
 */

/*
 * One-pass quantize + pack for groups that are `group` contiguous channels of
 * one row (group-wise along D; batch and tokens not reduced).  Performs
 * VAR_Q/quant.py:112-121 (scale, codes) fused with VAR_Q/pack_unpack.py:177-196
 * (pack); asym != 0 selects the min/max affine quantizer
 * (scale=(max-min)/(2^b-1), zp=qmin-round(min/scale)).
 *   x        [n_rows, c] row-major, dtype x_dtype (n_rows = n0*n1*n2 of rowmap)
 *   words    [out_rows, c*bits/32] int32
 *   scale,zp [out_rows, c/group] fp32 (zp may be NULL when asym == 0)
 *   host_rowmap  NULL = dense (output row == input row), else 8 int64 as above
 *   slot     device int32 table for slot_dim, or NULL
 * Requires bits in {2,4,8}, c % 8 == 0, c*bits % 32 == 0, group % 8 == 0,
 * c % group == 0 and group/8 a power of two <= 64.
 */
int varq_quant_pack_rows(const void *x, int x_dtype, int64_t n_rows, int c, int group, int bits,
                         int asym, float eps, const int64_t *host_rowmap, const int32_t *slot,
                         int32_t *words, float *scale, float *zp, void *stream);

/*
 * The same for two tensors of one shape in one launch -- K and V of a cache step, which
 * the reference quantizes one after the other (VAR/models/basic_var.py:146-147,
 * Infinity/infinity/models/basic.py:329-330).  Row map and slot table are shared; each
 * tensor has its own outputs.  Results are those of two varq_quant_pack_rows calls.
 */
int varq_quant_pack_rows2(const void *x0, const void *x1, int x_dtype, int64_t n_rows, int c, int group,
                          int bits, int asym, float eps, const int64_t *host_rowmap, const int32_t *slot,
                          int32_t *words0, float *scale0, float *zp0, int32_t *words1, float *scale1,
                          float *zp1, void *stream);

/*
 * General quantizer for the six grouping methods of VAR_Q/quant.py:75-95 and
 * any other reduce set: a group is every element sharing the indices of the
 * dims NOT in reduce_mask (bit d set = dim d reduced).  Two phases: group
 * min/max into `workspace`, then scale/zp and codes (VAR_Q/quant.py:112-121).
 *   x       [shape[0..3]] contiguous
 *   scale   [n_groups] fp32 in the order of the kept dims; zp likewise or NULL
 *   words   packed output [rows, ceil(c/(32/bits))] or NULL
 *   codes   int8 output [rows, c] or NULL (the pack_to_int32=False mode,
 *           VAR_Q/quant.py:174-175).  At least one of words/codes is non-NULL.
 *   host_out_map  NULL: output rows are the input rows.  Else 3 host int64
 *           {rows per block, extra rows per block, first row}: input row r is
 *           written to output row r + (r / rows_per_block) * extra + first, which
 *           puts a step straight into its tokens of a larger cache buffer instead
 *           of the torch.cat of VAR_Q/quant.py:200-201 -- a [B,H,n,c] step at token
 *           len of a [B,H,cap,..] buffer is {n, cap - n, len}, a [B,n,H,c] step in
 *           a [B,cap,H,..] buffer {n*H, (cap - n)*H, len*H}.
 *   workspace  >= varq_quant_workspace_bytes(...) bytes, any contents
 *   scale, zp and workspace are 16-byte aligned when the channel dim is kept and c is a
 *   multiple of 8 (those kernels move eight adjacent groups' parameters in 16-byte pieces);
 *   4-byte aligned otherwise
 * bits in 2..8 when only codes are requested, {2,4,8} when words are.
 */
size_t varq_quant_workspace_bytes(const int64_t *host_shape4, int reduce_mask);
int varq_quant_pack(const void *x, int x_dtype, const int64_t *host_shape4, int reduce_mask, int bits,
                    int asym, float eps, int32_t *words, int8_t *codes, float *scale, float *zp,
                    const int64_t *host_out_map, void *workspace, size_t workspace_bytes, void *stream);
/*
 * The same for two tensors of one shape and dtype with separate outputs and a shared output
 * map -- K and V of a step, which the reference quantizes one after the other
 * (Infinity/infinity/models/basic.py:329-330) -- in the same three launches.  The workspace
 * holds 2 * varq_quant_workspace_bytes(...) bytes.  Results are those of two varq_quant_pack calls.
 */
int varq_quant_pack2(const void *x0, const void *x1, int x_dtype, const int64_t *host_shape4, int reduce_mask,
                     int bits, int asym, float eps, int32_t *words0, int8_t *codes0, float *scale0, float *zp0,
                     int32_t *words1, int8_t *codes1, float *scale1, float *zp1,
                     const int64_t *host_out_map, void *workspace, size_t workspace_bytes, void *stream);

/*
 * varq_quant_pack for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart
 * in the reference.  Same arguments and results as varq_quant_pack, without a workspace:
 * the partial min/max and the group parameters go through a static device array of
 * VARQ_STATIC_SCRATCH_BYTES that each GPU the library runs on holds until the process
 * ends.  Calls no hipMalloc/hipFree and no allocating routine.  A shape and grouping
 * whose varq_quant_workspace_bytes exceeds the array is rejected with VARQ_ERR_WORKSPACE
 * (the six methods of VAR_Q/quant.py:75-95 need at most 8 MiB at the benchmark shapes).
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams,
 * two threads) race; calls ordered on one stream do not.
 * The address of a device's copy is looked up once per device, by the first call of either
 * function below with that device current.  That lookup is a runtime query, so it has to happen
 * outside graph capture: call varq_quant_static_scratch_bytes() (or the entry point itself) once
 * on each device before capturing.  Recorded into a graph, the entry point is kernel launches only.
 */
#define VARQ_STATIC_SCRATCH_BYTES (16u << 20)
size_t varq_quant_static_scratch_bytes(void);
int varq_quant_pack_static(const void *x, int x_dtype, const int64_t *host_shape4, int reduce_mask, int bits,
                           int asym, float eps, int32_t *words, int8_t *codes, float *scale, float *zp,
                           const int64_t *host_out_map, void *stream);

/* VAR_Q/pack_unpack.py:107-134 (and its CPU twin 177-196): int8 codes [rows,c]
 * -> int32 words [rows, ceil(c*bits/32)], zero padding in the last word. */
int varq_pack(const int8_t *codes, int64_t rows, int c, int bits, int32_t *words, void *stream);

/* VAR_Q/pack_unpack.py:136-162 (and 198-211): words -> sign-extended int8
 * codes [rows, c]. */
int varq_unpack(const int32_t *words, int64_t rows, int c, int bits, int8_t *codes, void *stream);

/*
 * Unpack + dequantize in one pass: VAR_Q/quant.py:216-224 (unpack, then
 * q.float()*scale, 123-124), with the affine form (q - zp)*scale when zp is
 * given.  The scale of element (i0,i1,i2,ch) of the [n0,n1,n2,c] code tensor
 * is scale[i0*ss[0] + i1*ss[1] + i2*ss[2] + (ch/group)*ss[3]] (strides in
 * elements, 0 = broadcast), so every layout the quantizer produces -- expanded
 * per-step scales, per-token group scales, per-head tables -- is addressed
 * without materializing it.
 *   words  packed codes, or codes_i8 unpacked int8 codes (exactly one non-NULL)
 *   in_row_stride  rows between consecutive i1 blocks is n2 unless the input
 *                  is a window of a larger cache: host_in_rowmap as above maps
 *                  (i0,i1,i2) to the INPUT row (NULL = dense)
 *   out    [n0*n1*n2, c] dense, dtype out_dtype
 */
int varq_dequant(const int32_t *words, const int8_t *codes_i8, const float *scale, const float *zp,
                 const int64_t *host_shape4, const int64_t *host_scale_strides4, int group, int bits,
                 const int64_t *host_in_rowmap, void *out, int out_dtype, void *stream);

/*
 * Fused dequant flash-attention (no counterpart in the reference, which
 * dequantizes the whole cache to fp32 and calls an external attention backend:
 * VAR_Q/quant.py:216-230, VAR/models/basic_var.py:156-162,
 * Infinity/infinity/models/basic.py:339-351).
 *
 *   out[b,h,i,:] = softmax_j( softmax_scale * q[b,h,i,:] . K[b,h,j,:] + mask(i,j) ) V[b,h,j,:]
 *   K = (k_codes - k_zp) * k_scale,  V likewise, never materialized.
 *
 *   q, out     [B, Hq, Lq, D] of io_dtype: VARQ_BF16 (the Infinity path, bf16 autocast:
 *              Infinity/tools/run_infinity.py:519) or VARQ_F16 (the VAR path, fp16 autocast:
 *              scripts/inference_multi_VAR.py:123, VAR/models/basic_var.py:157-158).  It is
 *              also the type dequantized K and V are rounded to and the type of the MFMA
 *              operands; accumulation is fp32 either way.  VARQ_F16 needs D = 64 (the head
 *              dim of every VAR model).
 *   operand_form  one of varq_attn_form (above)
 *   k_words    int32 [B, Hkv, Lk_stride, D*k_bits/32]; only rows < Lk are read
 *   k_scale/zp fp32  [B, Hkv, Lk_stride, D/k_group]   (zp NULL = symmetric)
 *   v_*        same for V
 *   head_map   device int32 [Hkv]: q/out head served by packed head slot s, or
 *              NULL for identity (then Hkv == Hq).  One launch per bit-width
 *              class serves a cache with mixed per-head bit-widths.
 *   kv_limit   device int32 [Lq]: query i sees keys j < kv_limit[i]
 *              (block-causal next-scale mask of VAR/models/var.py:110-114,
 *              limit = end of the query's own scale); NULL = all Lk visible.
 *              A query whose limit is 0 sees no key and gets zeros.
 *   Lq == 0    nothing is done (q and out may be NULL then); Lq > 0 with
 *              Lk == 0 is VARQ_ERR_INVALID (no keys to attend).
 *   layout     VARQ_LAYOUT_BHLC: the shapes above.  VARQ_LAYOUT_BLHC: q, out
 *              [B, Lq, Hq, D], words [B, Lk_stride, Hkv, D*bits/32], scales
 *              [B, Lk_stride, Hkv, D/group] -- the layout of the reference's
 *              flash-attention call (VAR/models/basic_var.py:127-131,157-158) and the
 *              default qkv_format of its quantizer.  VARQ_LAYOUT_BHLC_OUT_BLHC: q and
 *              the cache as VARQ_LAYOUT_BHLC, out [B, Lq, Hq, D], which is how the
 *              attention modules hand the result to their output projection
 *              (VAR/models/basic_var.py:160, Infinity/infinity/models/basic.py:347):
 *              no transposing copy behind the call.
 *   workspace, workspace_bytes, splits
 *              A launch with few query blocks over a long cache (a small batch, a
 *              step of a few hundred queries) leaves compute units idle or ends in a
 *              short last round.  The keys of each query block can be shared out over
 *              up to 8 workgroups; their partial results (fp32) pass through the
 *              workspace and a second kernel combines them.  splits = 0: the library
 *              decides, and uses no more shares than the workspace holds (none
 *              without a workspace) -- with at most 64 queries over at least 1024 keys
 *              (D = 128, one scale group per key, bf16) it takes a kernel of its own for
 *              that regime, whose wavefronts all serve the same 32 queries on different
 *              keys, with up to 64 shares; 1: never; 2..8: exactly that many (an error if
 *              the workspace is too small).  varq_fused_attn_workspace_bytes gives the
 *              size for a shape (0 when the library would not share the keys out);
 *              device memory, 16-byte aligned, used only during the call's kernels.
 * Requires D in {64,128}, bits in {2,4,8}, k_group/v_group in {32,64,128}
 * dividing D.
 */
size_t varq_fused_attn_workspace_bytes(int B, int Hkv, int Lq, int Lk, int D, int nseg, int splits);
/* Over how many workgroups varq_fused_attn shares the keys of a query block out when that is left
 * to it (splits = 0) and the workspace has room; 1 = not at all.  (A report for callers and
 * benchmarks; no counterpart in the reference.) */
int varq_fused_attn_key_shares(int B, int Hkv, int Lq, int Lk, int D, int k_group, int v_group);
int varq_fused_attn(const void *q, void *out,
                    const int32_t *k_words, const float *k_scale, const float *k_zp, int k_bits, int k_group,
                    const int32_t *v_words, const float *v_scale, const float *v_zp, int v_bits, int v_group,
                    int B, int Hq, int Hkv, const int32_t *head_map,
                    int Lq, int Lk, int Lk_stride, int D,
                    const int32_t *kv_limit, float softmax_scale, int layout, int io_dtype, int operand_form,
                    void *workspace, size_t workspace_bytes, int splits, void *stream);

/*
 * The same attention over a cache quantized per (head, channel), the layout of the
 * reference's G_SCALE_HEAD_DIM and G_HEAD_DIM methods (scale of shape [1,H,1,c],
 * VAR_Q/quant.py:84-88,112-116; G_SCALE_HEAD_DIM is the method of the shipped JSON rules)
 * and of their affine per-head-per-dim extension:
 *   K[b,h,j,d] = k_chan_scale[h,d] * (k_codes[b,h,j,d] - k_chan_zp[h,d]),  V likewise.
 * A scalar scale (G_TENSOR, G_SCALE) is the table filled with it.
 * A cache that the reference's append methods filled step by step
 * (VAR_Q/quant.py:196-201: every step is quantized with its own scale, expanded over the
 * step's tokens and concatenated) has one table per step: keys
 * [host_seg_end[s-1], host_seg_end[s]) use table s, the last segment ends at Lk.
 *   k_chan_scale, k_chan_zp, v_chan_scale, v_chan_zp
 *                        fp32 [nseg, Hkv, D]; zero-points NULL = symmetric.  With one
 *                        segment k_chan_zp may be NULL for an affine K as well: it shifts
 *                        every logit of a query by the same amount, which the softmax cancels
 *                        (K is then offset per channel before it is rounded to bf16)
 * K and V are dequantized with the tables of each key's segment as tiles enter LDS,
 * (code - zp) * scale in fp32 rounded to io_dtype (bf16 or fp16, as in varq_fused_attn): the
 * operands of the reference's attention after dequant_all (VAR_Q/quant.py:216-224) and the
 * downcast of its attention call.
 *   nseg, host_seg_end   1..16 segments; host int32 [nseg] (may be NULL when nseg == 1)
 *   everything else as in varq_fused_attn; one bit-width for K and V.
 */
int varq_fused_attn_channel(const void *q, void *out,
                            const int32_t *k_words, const float *k_chan_scale, const float *k_chan_zp,
                            const int32_t *v_words, const float *v_chan_scale, const float *v_chan_zp,
                            int nseg, const int32_t *host_seg_end,
                            int bits, int B, int Hq, int Hkv, const int32_t *head_map,
                            int Lq, int Lk, int Lk_stride, int D,
                            const int32_t *kv_limit, float softmax_scale, int layout, int io_dtype,
                            void *workspace, size_t workspace_bytes, int splits, void *stream);

/*
 * Producer side of the quantized cache in one pass (an extension: the reference does
 * this as separate tensor expressions before calling its quantizer,
 * Infinity/infinity/models/basic.py:316-330 with apply_rotary_emb at :103-123, and
 * VAR/models/basic_var.py:137-147).  Reads the qkv projection output
 * [B, L, 3, H, c] once and
 *   - writes q: optionally l2-normalised (x / max(|x|_2, norm_eps)) and multiplied by
 *     q_scale_mul[h], optionally rotated (pairs (2i, 2i+1) by the angle whose cos/sin
 *     are rope_cos/sin[token_start + l][i]), as bf16 [B, H, L, c];
 *   - quantizes k (normalised, rotated) and v group-wise (as varq_quant_pack_rows) into
 *     their cache rows: input row (b, l, h) goes to the row the map gives for
 *     (n0, n1, n2) = (B, L, H).
 * With a slot table over the heads (slot_dim = 2: one call per bit-width class of a
 * mixed cache) a head whose slot is negative is left out altogether, its q included:
 * the calls of the classes share out the heads and between them write all of q.
 * c in {32, 64, 128}; group a power of two in [8, c] (>= 16 for 2-bit codes).
 */
int varq_qkv_prepare_append(const void *qkv, int x_dtype, int B, int L, int H, int c,
                            const float *q_scale_mul, int l2norm, float norm_eps,
                            const float *rope_cos, const float *rope_sin, int token_start,
                            void *q_out, int group, int bits, int asym, float eps,
                            const int64_t *host_rowmap, const int32_t *slot,
                            int32_t *k_words, float *k_scale, float *k_zp,
                            int32_t *v_words, float *v_scale, float *v_zp, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* VARQ_H */
