/*
 * omni_dit.h — flat C ABI of libomni_dit_hip.so: the MI355X (gfx950) kernels under the per-step
 * DiT transformer-block forward of vLLM-Omni's diffusion stack.
 *
 * Conventions
 *   - Every pointer except `stream` is a DEVICE pointer owned by the caller. No entry point
 *     allocates or frees device memory, and none synchronises except odit_linear_tune (a set-up
 *     call that times kernels); all work is enqueued on `stream` (a hipStream_t; NULL = the legacy
 *     default stream).
 *   - Tensors are row-major with the innermost dimension contiguous. Strides are in ELEMENTS.
 *   - `dtype` is one of ODIT_BF16 / ODIT_F16 / ODIT_F32 and names the element type of the activation
 *     tensors. Arithmetic inside every kernel is fp32.
 *   - Return value: 0 on success, a negative ODIT_E* code on failure; odit_last_error() then returns a
 *     thread-local, NUL-terminated description. Argument errors are detected on the host BEFORE any
 *     launch, so a failing call enqueues nothing.
 *   - Re-entrant; the state kept between calls is thread-local (the error string, and in odit_linear the
 *     library handle with the matmul descriptors of the problems seen so far) or process-wide behind a
 *     lock or an atomic (each device's compute-unit count, the record of which engine a tuning call found
 *     faster for a problem, the launch counter that ticket words in caller scratch are stamped with).
 *
 * The reference (Flink-ddd/vllm-omni) is pure Python and has no FFI of its own for this path; each
 * entry point below replaces the third-party kernel call(s) made at the cited reference lines.
 */
#ifndef OMNI_DIT_H_
#define OMNI_DIT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ODIT_VERSION 200 /* major*10000 + minor*100 + patch */

enum odit_dtype { ODIT_BF16 = 0, ODIT_F16 = 1, ODIT_F32 = 2 };

enum odit_status {
  ODIT_OK = 0,
  ODIT_EINVAL = -1,   /* bad shape / stride / alignment / null pointer            */
  ODIT_ENOTSUP = -2,  /* valid request this build has no kernel for               */
  ODIT_ELAUNCH = -3,  /* hipLaunchKernel / hipGetLastError reported a failure     */
  ODIT_EWORKSPACE = -4 /* caller workspace too small                              */
};

/* Flag bits shared by the elementwise entry points. */
#define ODIT_FLAG_REF_ROUNDING 1u /* round intermediates to `dtype` at the points where the reference's
                                     op-by-op torch path does (makes bf16 results track the reference
                                     bit-for-bit up to reduction order); default is one final rounding */
#define ODIT_FLAG_NEOX 2u         /* rotary: rotate (i, i+rot/2) pairs instead of (2i, 2i+1)            */

int odit_version(void);
const char* odit_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * K1  joint (text+image) non-causal flash attention:  o = softmax(q k^T * scale [+ key mask]) v
 *
 * Replaces torch.nn.functional.scaled_dot_product_attention at
 *   vllm_omni/diffusion/attention/backends/sdpa.py:82-90
 * and aiter/flash-attn `flash_attn_func` at
 *   vllm_omni/diffusion/attention/backends/flash_attn.py:105-111, utils/fa.py:24-32
 * behind AttentionImpl.forward_hip (backends/abstract.py:132-140).
 *
 * q [B,Sq,H,D], k,v [B,Sk,Hkv,D], o [B,Sq,H,D]; layout BSHD as the reference passes them; each
 * tensor gives strides for (batch, seq, head); the D axis must be contiguous, every stride a
 * multiple of 8 elements and every base pointer 16-byte aligned. H % Hkv == 0 (grouped KV).
 * key_mask: NULL, or uint8 [B,Sk] (row stride Sk); keys with mask == 0 are excluded, matching the
 *   [B,Sk] boolean key-padding mask of flash_attn.py:80-102. A row whose keys are all excluded
 *   returns zeros.
 * lse: NULL, or float [B,H,Sq] receiving log(sum exp(scale*q.k)) per row (natural log).
 * dtype: ODIT_BF16 or ODIT_F16 (fp32 never reaches a backend: attention/layer.py:134-140).
 * D in {64, 128}.
 */
int odit_attn_fwd(const void* q, const void* k, const void* v, void* o, const uint8_t* key_mask,
                  float* lse, int B, int Sq, int Sk, int H, int Hkv, int D,
                  const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t v_strides[3], const int64_t o_strides[3], float scale, int dtype,
                  void* stream);

/* Extended form of odit_attn_fwd with three optional additions.
 *
 * Values in two tensors: with v_tail != NULL, key rows [0, k_split) take their values from `v` and rows
 * [k_split, Sk) from `v_tail` (row r -> v_tail row r - k_split); k_split is a multiple of 64, both share
 * the row stride (v_tail_strides[1] == v_strides[1]), batch and head strides are their own. Lets the
 * joint attention read V straight out of the two fused-QKV projection outputs: the value halves of
 * torch.cat([txt_value, img_value]) (qwen_image_transformer.py:603-606, flux_transformer.py:200-208)
 * are never copied. Keys still come as one tensor (they are rewritten by norm + rotary anyway).
 *
 * Two outputs: with o_tail != NULL, query rows [0, q_split) are written to `o` (row r -> o row r) and
 * rows [q_split, Sq) to `o_tail` (row r -> o_tail row r - q_split), each with its own (batch, seq,
 * head) strides. Replaces the two slices joint_hidden_states[:, :seq_len_txt] / [:, seq_len_txt:] of
 * qwen_image_transformer.py:654-656 (flux_transformer.py:217-219), whose strided views otherwise force
 * a copy in front of each output projection.
 *
 * Scratch: `workspace` (device memory, 16-byte aligned, workspace_bytes >=
 * odit_attn_fwd_workspace_bytes for the same shape, contents irrelevant before and after) lets the
 * kernel cut the last, partly filled round of workgroups into key ranges that run side by side and
 * are merged by a second launch; it is used when that last round would fill at most a quarter of the
 * GPU, where the unsplit launch leaves most of the GPU idle. NULL = never split. Results with and
 * without scratch agree to rounding (the merge re-associates the key sum); for given shapes and device
 * the partition is fixed, so repeated calls are bit-identical. No counterpart in the reference.
 * The first 1024 bytes of the scratch belong to a measurement mode (ODIT_ATTN_PERSISTENT=1 and
 * ODIT_ATTN_WAVES=4 in the environment when the library makes its first attention launch: as many workgroups
 * of 4 wavefronts as run at once, each drawing unit after unit from ticket words there). That mode alone needs those bytes zero before the first
 * call that uses the buffer and leaves them zero; no default launch reads or writes them.
 *
 * v_tail == NULL, o_tail == NULL and workspace == NULL behaves exactly like odit_attn_fwd.
 */
int odit_attn_fwd_ex(const void* q, const void* k, const void* v, const void* v_tail, int k_split, void* o,
                     void* o_tail, int q_split, const uint8_t* key_mask, float* lse, int B, int Sq, int Sk,
                     int H, int Hkv, int D, const int64_t q_strides[3], const int64_t k_strides[3],
                     const int64_t v_strides[3], const int64_t v_tail_strides[3], const int64_t o_strides[3],
                     const int64_t o_tail_strides[3], float scale, int dtype, void* workspace,
                     size_t workspace_bytes, void* stream);

/* Scratch bytes odit_attn_fwd_ex can use for this shape on the current device (0 = none needed). */
size_t odit_attn_fwd_workspace_bytes(int B, int Sq, int Sk, int H, int D);

/* Which kernels odit_attn_fwd_ex launches for a problem, as text: "<kernel> units=<workgroups>" per
 * launch, joined by "; " (the kernel names are the ones a profiler reports). k_seq_stride / v_seq_stride
 * are the sequence strides of k and v in elements; with_workspace says whether scratch will be given.
 * Returns the number of launches, or a negative status. Host-only: enqueues nothing. No counterpart in the
 * reference; for tests and for benchmarks that must name the kernel they time.
 */
int odit_attn_fwd_plan(int B, int Sq, int Sk, int H, int D, int64_t k_seq_stride, int64_t v_seq_stride,
                       int with_workspace, char* text, size_t text_bytes);

/* ---------------------------------------------------------------------------------------------
 * K2  fused QK-RMSNorm + rotary embedding + scatter into the joint [txt;img] sequence.
 *
 * Replaces, in one pass over a fused-QKV projection output:
 *   vLLM RMSNorm(head_dim) x2       vllm_omni/diffusion/models/qwen_image/qwen_image_transformer.py:588-591
 *   RotaryEmbedding.forward x2      vllm_omni/diffusion/layers/rope.py:108-159 (interleaved: rope.py:12-36)
 *   torch.cat([txt, img], dim=1) x3 qwen_image_transformer.py:603-606
 * and, with norm_mode = ODIT_NORM_ROW, Wan's whole-row fp32 RMSNorm + apply_rotary_emb_wan
 *   vllm_omni/diffusion/models/wan2_2/wan2_2_transformer.py:34-56, 59-89, 406-420.
 *
 * q_in/k_in/v_in: [B,S,H,D] views (typically slices of one [B,S,3*H*D] GEMM output) addressed by
 *   in_strides = (batch, seq) strides in elements, shared by the three; heads are D apart.
 *   k_in and v_in may be NULL (then only q is processed); v is copied unchanged.
 * q_out/k_out/v_out: [B,S_total,H,D] dense joint buffers; row s of the input lands in row
 *   out_seq_offset + s. May alias the inputs only if layouts coincide exactly.
 * wq, wk: RMSNorm weights, float32 or `dtype` per w_dtype; [D] for ODIT_NORM_HEAD, [H*D] for
 *   ODIT_NORM_ROW; NULL = weight of ones. Ignored for ODIT_NORM_NONE.
 * cos, sin: float32 [S, rot/2] tables (row stride rot/2), NULL = no rotation (identity).
 *   rot <= D, rot % 8 == 0. Pair (x[2i], x[2i+1]) -> (x0*c - x1*s, x1*c + x0*s); with
 *   ODIT_FLAG_NEOX pair (x[i], x[i+rot/2]).
 * With ODIT_FLAG_REF_ROUNDING: normalised value rounded to `dtype` before the weight multiply
 *   (vLLM RMSNorm order; skipped for ODIT_NORM_ROW whose reference keeps fp32), cos/sin rounded to
 *   `dtype` (qwen_image_transformer.py:593-596) and the rotation evaluated in `dtype` steps.
 */
enum odit_norm_mode { ODIT_NORM_NONE = 0, ODIT_NORM_HEAD = 1, ODIT_NORM_ROW = 2 };

int odit_qknorm_rope(const void* q_in, const void* k_in, const void* v_in, void* q_out, void* k_out,
                     void* v_out, const void* wq, const void* wk, const float* cos, const float* sin,
                     int B, int S, int H, int D, int rot, const int64_t in_strides[2],
                     int out_seq_offset, int S_total, float eps, int norm_mode, int w_dtype,
                     int dtype, unsigned flags, void* stream);

/* Two odit_qknorm_rope problems that fill different rows of the same joint buffers, in ONE launch: the text
 * rows and the image rows of a dual-stream block (qwen_image_transformer.py:588-606, where the reference
 * normalises and rotates the two streams separately and concatenates them). Element i of every array belongs to
 * problem i; in_strides = {batch0, seq0, batch1, seq1}. Both problems share B, H, D, rot, S_total, eps,
 * norm_mode, the dtypes and the flags, and take the same optional operands (k, v, rotary tables). With
 * ODIT_NORM_ROW, or when one problem is empty, the call makes one launch per problem. */
int odit_qknorm_rope_pair(const void* const q_in[2], const void* const k_in[2], const void* const v_in[2],
                          void* q_out, void* k_out, void* v_out, const void* const wq[2],
                          const void* const wk[2], const float* const cos[2], const float* const sin[2],
                          int B, const int S[2], int H, int D, int rot, const int64_t in_strides[4],
                          const int out_seq_offset[2], int S_total, float eps, int norm_mode, int w_dtype,
                          int dtype, unsigned flags, void* stream);

/* ---------------------------------------------------------------------------------------------
 * K3  fused LayerNorm (no affine, or fp32 affine) + adaLN shift/scale modulation:
 *        out = LN(x) * (1 + scale) + shift
 *
 * Replaces nn.LayerNorm + mul + add in AdaLayerNorm.forward_native
 *   vllm_omni/diffusion/layers/adalayernorm.py:23-60, 102-110
 * (same arithmetic: QwenImageTransformerBlock._modulate qwen_image_transformer.py:710-744;
 *  Flux norm2 + inline modulate flux_transformer.py:292-293; Wan FP32LayerNorm + modulate
 *  wan2_2_transformer.py:659, 668-670).
 *
 * x, out: [B,S,C], x_strides/out_strides = (batch, seq) strides; C contiguous.
 * shift, scale: element (b, s, c) at ptr[b*mod_stride_b + s*mod_stride_s + c]; NULL = 0. Type per
 *   mod_dtype (`dtype` or ODIT_F32). mod_stride_s = 0 is one row per batch entry; non-zero is one row
 *   per token (Wan per-token timesteps, temb [B,S,6,C], wan2_2_transformer.py:641-652).
 *   `gate` is not touched here: the caller returns it as a view.
 * shift_bias, scale_bias: NULL or float32 [C] added to the shift / scale row in fp32 (Wan's
 *   scale_shift_table + temb.float(), wan2_2_transformer.py:643-645, 654-656, without forming the sum
 *   in memory).
 * index: NULL, or int32 [B,S] (row stride S): token (b,s) uses modulation row b when index == 0 and
 *   row b + B otherwise (adalayernorm.py:31-54); needs mod_stride_s == 0.
 * ln_weight, ln_bias: NULL or float32 [C] (elementwise-affine LayerNorm, applied before modulation).
 */
int odit_adaln_modulate(const void* x, void* out, const void* shift, const void* scale,
                        const int32_t* index, const float* ln_weight, const float* ln_bias,
                        const float* shift_bias, const float* scale_bias, int B, int S, int C,
                        const int64_t x_strides[2], const int64_t out_strides[2],
                        int64_t mod_stride_b, int64_t mod_stride_s, float eps, int mod_dtype,
                        int dtype, unsigned flags, void* stream);

/* odit_adaln_modulate for two tensors of the same batch and width in ONE launch: img_norm1 and txt_norm1
 * (or img_norm2 and txt_norm2) of a dual-stream block, which the reference calls one after the other
 * (qwen_image_transformer.py:770-773, 798, 804). One modulation row per batch entry (no index, no
 * LayerNorm affine, no tables); element i of every array belongs to problem i, x_strides / out_strides =
 * {batch0, seq0, batch1, seq1}, mod_stride_b[i] the row stride of shift[i] / scale[i]. */
int odit_adaln_modulate_pair(const void* const x[2], void* const out[2], const void* const shift[2],
                             const void* const scale[2], int B, const int S[2], int C,
                             const int64_t x_strides[4], const int64_t out_strides[4],
                             const int64_t mod_stride_b[2], float eps, int mod_dtype, int dtype,
                             unsigned flags, void* stream);

/* ---------------------------------------------------------------------------------------------
 * K4  gated residual:  out = h + gate * y     (gate broadcast over the sequence, or per token)
 *
 * Replaces the torch mul + add at qwen_image_transformer.py:794-795, 801, 806
 * (Flux flux_transformer.py:289-290, 299-300, 362-364; Wan wan2_2_transformer.py:661, 673 with
 *  fp32 gate). gate == NULL means gate of ones (plain residual, wan2_2_transformer.py:666).
 *
 * h, y, out: [B,S,C] with (batch, seq) strides; out may alias h.
 * gate element (b,s,c) at gate[b*gate_strides[0] + s*gate_strides[1] + c]; type per gate_dtype.
 * gate_bias: NULL or float32 [C] added to the gate in fp32 (Wan's scale_shift_table row + per-token
 *   temb row, wan2_2_transformer.py:643-652); with gate == NULL the table alone is the gate.
 */
int odit_gated_residual(const void* h, const void* y, const void* gate, const float* gate_bias,
                        void* out, int B, int S, int C, const int64_t h_strides[2],
                        const int64_t y_strides[2],
                        const int64_t out_strides[2], const int64_t gate_strides[2], int gate_dtype,
                        int dtype, unsigned flags, void* stream);

/* ---------------------------------------------------------------------------------------------
 * K5  TeaCache relative-L1 reduction, per batch row:
 *        sums[b] = ( sum_i |cur[b,i] - prev[b,i]| , sum_i |prev[b,i]| )
 *
 * Replaces the six torch kernels of
 *   vllm_omni/diffusion/cache/teacache/hook.py:214-221
 * ((cur-prev).abs().mean() / (prev.abs().mean() + 1e-8)); the host divides and applies the
 * polynomial. With ODIT_FLAG_REF_ROUNDING the difference is rounded to `dtype` before abs(), as
 * torch does for a bf16 subtraction. One launch. Deterministic: every workgroup leaves an fp32 partial
 * of a fixed slice, and the workgroup that finishes a row last adds the row's partials in fp64 in slot
 * order, so the result does not depend on which one that is.
 *
 * cur, prev: [B, n] with row strides cur_stride / prev_stride (elements); n % 8 == 0 not required.
 * sums: double [B,2] on the device.
 * workspace: device scratch of at least odit_rel_l1_workspace_bytes(B, n) bytes, 16-byte aligned: a
 *   region of fixed size (568 KiB, whatever B is) with one 64-bit ticket word per row and the group words that
 *   rows of many workgroups draw from first, then the partials.
 *   ZERO-FILL IT ONCE after allocating it (hipMemsetAsync, or a fill kernel under graph capture) and do
 *   not write it afterwards. A ticket word is (launch number << 16 | tickets drawn); every launch first
 *   raises its rows' words to its own number, which is larger than any earlier launch's, and the last
 *   workgroup of a row puts the word back to zero. One zeroed workspace therefore serves any number of
 *   later calls of any (B, n) it is large enough for, also after a launch that did not finish (its stale
 *   words are overridden), and a call recorded into a HIP graph can be replayed. Calls that share a
 *   workspace must not overlap (same stream, or ordered by events).
 */
size_t odit_rel_l1_workspace_bytes(int B, int64_t n);
int odit_rel_l1(const void* cur, const void* prev, double* sums, void* workspace,
                size_t workspace_bytes, int B, int64_t n, int64_t cur_stride, int64_t prev_stride,
                int dtype, unsigned flags, void* stream);

/* odit_rel_l1 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same arguments and bit-identical
 * sums, without the workspace: the ticket words and partials live in an array built into the library's
 * device image, 2560 bytes per GPU the library is used on, held until the process ends. It calls no
 * allocating routine. Limit: B <= 64 rows (any n); more returns ODIT_EWORKSPACE and enqueues nothing.
 * Two launches: a fill kernel puts the ticket words to zero (a kernel, not a memset, so the call can be
 * captured; whatever an earlier call left in the array, also one that never finished, is gone), then the reduction. Every call on a GPU shares that GPU's array: calls that may overlap on one GPU
 * (different streams without ordering, or several host threads) race and must be serialised by the caller.
 * The first call on each device looks the array's address up (hipGetSymbolAddress); make that call outside
 * graph capture.
 */
int odit_rel_l1_static(const void* cur, const void* prev, double* sums, int B, int64_t n, int64_t cur_stride,
                       int64_t prev_stride, int dtype, unsigned flags, void* stream);

/* Device address of that built-in array on the current device and its size (*bytes, may be NULL); NULL with
 * an error string when it cannot be looked up. No counterpart in the reference. For diagnostics and tests (a
 * test dirties the array to check that odit_rel_l1_static does not depend on what it holds); no caller of
 * odit_rel_l1_static needs it.
 */
void* odit_rel_l1_static_scratch(size_t* bytes);

/* ---------------------------------------------------------------------------------------------
 * Pointwise helpers on the block path.
 *
 * odit_gelu_tanh: out = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) over n contiguous elements;
 *   replaces F.gelu(approximate="tanh") at qwen_image_transformer.py:424.
 * odit_silu: out = x * sigmoid(x); replaces nn.SiLU at qwen_image_transformer.py:682-685, 699-702.
 */
int odit_gelu_tanh(const void* x, void* out, int64_t n, int dtype, void* stream);
int odit_silu(const void* x, void* out, int64_t n, int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Dense projection with the elementwise work done in the GEMM's epilogue:
 *     ODIT_EPI_NONE / ODIT_EPI_BIAS        out = x W^T (+ bias)
 *     ODIT_EPI_(BIAS_)GELU_TANH            out = gelu_tanh(x W^T (+ bias))
 *     ODIT_EPI_GATED_RESIDUAL              out = residual + gate * (x W^T + bias)
 *     ODIT_EPI_GATED_RESIDUAL_PRE          out = residual + gate * (x W^T) + bias, with float32 `gate` and a
 *                                          float32 `bias` the caller has already multiplied by the gate
 *                                          (NULL = none): no helper launch; for callers that form the
 *                                          gates of all blocks of a step at once
 *
 * Replaces, as one launch each (plus a [N]-sized helper launch for the gated form):
 *   ColumnParallelLinear + F.gelu(approximate="tanh")     qwen_image_transformer.py:399-424,
 *                                                          flux_transformer.py:30-45, wan2_2_transformer.py:92-109
 *   RowParallelLinear followed by `h + gate * y`           qwen_image_transformer.py:794-795, 801, 806,
 *                                                          flux_transformer.py:288-309, wan2_2_transformer.py:661, 673
 * Engines. hipBLASLt's MFMA kernels (a plain dense GEMM), set up so that bias, activation, gate and
 * residual ride in that kernel's epilogue, and two hand-written bf16 MFMA kernels (K a multiple of 64, N a
 * multiple of 8, 16-byte aligned rows): a stream-K kernel for 64 <= M <= 1024 rows (csrc/gemm_bf16.hip) that
 * keeps all CUs busy on few output tiles, and a tile kernel for more rows (csrc/gemm_bf16_tile.hip: 256 x 256
 * or 256 x 192 output tiles, one per workgroup). Both take one gate vector per group of rows in a single
 * launch (odit_linear_rows). A hand-written kernel runs where a tuning call found it faster or, untuned,
 * where its default rule says so (stream-K: K >= 2 N); the `flags` of odit_linear_rows can force either side.
 *
 * x [M,K] (row stride ldx), W [N,K] (row stride ldw: torch's nn.Linear weight, or a column range of
 * one), bias [N] or NULL, out [M,N] (row stride ldo). Gated form: residual [M,N] (row stride ldr; may be
 * `out` itself), gate [N] of `dtype` or float32 (gate_dtype), NULL = ones: one call per batch row when
 * the gate differs per batch row. dtype: ODIT_BF16, ODIT_F16 or ODIT_F32 (fp32 accumulation always).
 * workspace: device scratch, 256-byte aligned, for the library's split-K kernels, in the gated form two
 * float[N] vectors, and the hand-written kernel's tile counters and partial tiles;
 * odit_linear_workspace_bytes() is a size that suits every kernel. A workspace of that size must be
 * ZERO-FILLED ONCE before its first use and not written by the caller afterwards (the first 32 KB hold
 * the stream-K kernel's ticket words, stamped with the launch number like those of odit_rel_l1: every call
 * leaves them at zero, and what a launch that did not finish left there is overridden by the next one);
 * calls that share a workspace must not overlap in time (one workspace per stream). A smaller workspace goes to the library alone and rules the
 * hand-written kernel out; NULL restricts the choice to library kernels that need none (not allowed
 * for the gated form).
 *
 * odit_linear_tune launches every kernel the library offers for the problem, and the hand-written
 * kernel where it takes the problem, on the given buffers
 * (`out` is overwritten; this call synchronises with the stream), keeps the fastest library kernel for later
 * odit_linear calls with the same shape, strides, epilogue and dtype FROM THE SAME HOST THREAD, records
 * for the whole process whether the hand-written kernel beat it, and reports the winner's time. `flush` (optional device buffer, ideally larger than the last-level cache) is
 * overwritten before every timed launch so that each one starts from cold caches, as a projection
 * with its own weights does inside a model. Without tuning the library's own first choice is used.
 */
enum odit_epilogue {
  ODIT_EPI_NONE = 0,
  ODIT_EPI_BIAS = 1,
  ODIT_EPI_GELU_TANH = 2,
  ODIT_EPI_BIAS_GELU_TANH = 3,
  ODIT_EPI_GATED_RESIDUAL = 4,
  ODIT_EPI_GATED_RESIDUAL_PRE = 5
};

size_t odit_linear_workspace_bytes(void);

int odit_linear(const void* x, const void* w, const void* bias, void* out, const void* residual,
                const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int64_t ldr,
                int epilogue, int gate_dtype, int dtype, void* workspace, size_t workspace_bytes, void* stream);

int odit_linear_tune(const void* x, const void* w, const void* bias, void* out, const void* residual,
                     const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int64_t ldr,
                     int epilogue, int gate_dtype, int dtype, void* workspace, size_t workspace_bytes,
                     void* stream, int iters, void* flush, size_t flush_bytes, float* best_us);

/* odit_linear with one gate vector per group of rows_per_gate consecutive rows (the rows of one batch
 * row of a [B, S, N] activation): gate vector i, gate_stride elements after vector i - 1, scales rows
 * [i rows_per_gate, (i + 1) rows_per_gate); in the pre-scaled form `bias` is laid out the same way.
 * rows_per_gate = 0 is odit_linear. One launch when a hand-written kernel takes the problem, one
 * library launch per group of rows otherwise.
 * flags: 0 = choose as described above; ODIT_LINEAR_LIBRARY = hipBLASLt whatever the record says;
 * ODIT_LINEAR_HANDWRITTEN = the hand-written kernel for this row count (ODIT_ENOTSUP when it does not take
 * the problem). Per call: no process-wide switch exists.
 */
#define ODIT_LINEAR_LIBRARY 1u
#define ODIT_LINEAR_HANDWRITTEN 2u

int odit_linear_rows(const void* x, const void* w, const void* bias, void* out, const void* residual,
                     const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int64_t ldr,
                     int epilogue, int gate_dtype, int dtype, int rows_per_gate, int64_t gate_stride,
                     unsigned flags, void* workspace, size_t workspace_bytes, void* stream);

/* What odit_linear_rows would do with these arguments, without launching anything: *handwritten = 1 when
 * a hand-written kernel would run, *launches = kernel launches the call would make. */
int odit_linear_rows_plan(const void* x, const void* w, const void* bias, void* out, const void* residual,
                          const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int64_t ldr,
                          int epilogue, int gate_dtype, int dtype, int rows_per_gate, int64_t gate_stride,
                          unsigned flags, void* workspace, size_t workspace_bytes, int* handwritten, int* launches);

/* odit_linear_tune for the per-row-group form; *handwritten (may be NULL) = 1 when the hand-written kernel won. */
int odit_linear_rows_tune(const void* x, const void* w, const void* bias, void* out, const void* residual,
                          const void* gate, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, int64_t ldr,
                          int epilogue, int gate_dtype, int dtype, int rows_per_gate, int64_t gate_stride,
                          void* workspace, size_t workspace_bytes, void* stream, int iters, void* flush,
                          size_t flush_bytes, float* best_us, int* handwritten);

#ifdef __cplusplus
}
#endif
#endif /* OMNI_DIT_H_ */
