/*
 * hdit.h -- C ABI of the MI355X (gfx950) DiT denoise-step hot path.
 *
 * Every entry point takes plain device pointers, sizes and strides (in
 * elements), a HIP stream passed as void*, and returns 0 on success or a
 * negative HDIT_E* code.  No entry point allocates, frees, synchronises or
 * throws; work is enqueued on the given stream.  bf16 tensors are raw 16-bit
 * storage; "f32" pointers are IEEE binary32.
 *
 * The reference (PKU-DAIR/Hetu-DiT) is pure Python and has no FFI of its own:
 * each entry point below names the Python call site it replaces
 * (paths relative to hetu_dit/model_executor/diffusion_executor/ unless
 * stated otherwise).
 */
#ifndef HDIT_H
#define HDIT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HDIT_OK 0
#define HDIT_EINVAL (-1)      /* bad shape / stride / alignment / null pointer */
#define HDIT_EUNSUPPORTED (-2) /* shape outside what the kernels are built for */
#define HDIT_ELAUNCH (-3)     /* the HIP runtime refused the launch */
#define HDIT_ETOOLARGE (-4)   /* the problem needs more than a fixed-size internal buffer holds */

/* Version of this ABI; bumped when a struct below changes. */
int hdit_abi_version(void);
/* Static string describing the last HDIT_ELAUNCH on this thread ("" if none). */
const char* hdit_last_error(void);
/* Measurement aid without a counterpart in the reference: enqueues `slots`
 * one-wave workgroups (<= 1024; they spread over the CUs); workgroup i stores
 * four 64-bit values to out[4i..4i+3] (device memory, 8-byte aligned): the
 * shader-clock counter, the constant 100 MHz counter, the id of the XCD it ran
 * on, and the hardware id register (shader engine / array / CU in bits 8-15).
 * Every CU counts its own shader clock: two samples taken on the same CU around
 * the work being timed give the average shader clock the work ran at,
 * (d out[0]) / (d out[1]) x 100 MHz. */
int hdit_clock_sample(void* out, int slots, void* stream);
/* Second measurement aid, no counterpart in the reference: do the matrix pipe
 * and the vector ALU of a SIMD work side by side?  `workgroups` (<= 1024)
 * workgroups of 8 waves, one per CU; waves w and w + 4 share a SIMD.  Waves 0-3
 * run role_a and waves 4-7 role_b for `iters` iterations: nothing, 32
 * independent v_mfma_f32_32x32x16_bf16 per iteration (the matrix work of one
 * 64 x 64 x 64 attention tile), that tile's softmax VALU work (64 v_exp_f32, 32
 * packs, 32 pair sums, 32 v_max3, 64 subtractions), or both interleaved 1 : 7
 * in one instruction stream.  out (device, 8-byte aligned, workgroups * 16 + 1
 * 64-bit values): per wave the shader cycles and the 100 MHz ticks it took,
 * out[(16 g + 2 w)], out[16 g + 2 w + 1].  bench.py --probe coissue prints the
 * table. */
#define HDIT_PROBE_IDLE 0
#define HDIT_PROBE_MFMA 1
#define HDIT_PROBE_VALU 2
#define HDIT_PROBE_INTERLEAVED 3
int hdit_probe_coissue(int role_a, int role_b, int iters, int workgroups, void* out, void* stream);

/* ------------------------------------------------------------------------
 * Grouped bf16 GEMM with fused epilogue:  C = epilogue(A . B^T + bias)
 *
 * A [m, k] row-major (lda), B [n, k] row-major (ldb; an nn.Linear weight),
 * C [m, n] row-major (ldc); fp32 accumulation on MFMA.  Requirements:
 * k % 64 == 0, n % 8 == 0, lda/ldb/ldc/ldr % 8 == 0, every pointer 16-byte
 * aligned, m * lda and n * ldb below 2^31 elements, m * ldc and m * ldr below
 * 2^30.  Problems of one call may be spread over several kernel launches (one
 * per tile shape) on the given stream.  Up to
 * HDIT_GEMM_MAX_PROBLEMS problems share one launch (the image and text streams
 * of a joint block, or q|k|v|mlp of a fused projection).
 *
 * Replaces the nn.Linear calls at layers/attention_processor.py:688-695 (SD3
 * q/k/v + add_q/k/v), :844-846,:867-869 (Flux), :1054-1056 (CogVideoX),
 * :419-421,:294-295,:268 (out-projections, bias re-added at :428-447),
 * layers/feedforward.py:74-77 (MLP + output bias), and the diffusers block's
 * gated residual that consumes them (transformer_sd3.py:136-152).
 * ---------------------------------------------------------------------- */
#define HDIT_GEMM_MAX_PROBLEMS 16

#define HDIT_EPI_BIAS 0          /* C = acc + bias */
#define HDIT_EPI_BIAS_GELU 1     /* C = gelu_tanh(acc + bias) */
#define HDIT_EPI_GATE_RESIDUAL 2 /* C = resid + gate[row / rows_per_batch] * (acc + bias) */
#define HDIT_EPI_MODE_MASK 0xf
/* Flags ORed into `epilogue` with HDIT_EPI_GATE_RESIDUAL: the residual stream of a
 * block stack carried in fp32 between the gated residuals, so that its rounding
 * does not accumulate over 24+ blocks.  With HDIT_EPI_RESID_F32 `resid` is f32
 * [m, n] (ldr in f32 elements), with HDIT_EPI_OUT_F32 `c` is f32 [m, n] (ldc in
 * f32 elements); the sum resid + gate * (.) is formed in fp32 either way. */
#define HDIT_EPI_RESID_F32 0x10
#define HDIT_EPI_OUT_F32 0x20

typedef struct hdit_gemm_problem {
  const void* a;     /* bf16 [m, k] */
  const void* b;     /* bf16 [n, k] */
  void* c;           /* bf16 [m, n] (f32 with HDIT_EPI_OUT_F32) */
  const void* bias;  /* bf16 [n] or NULL */
  const void* resid; /* bf16 [m, n] (ldr; f32 with HDIT_EPI_RESID_F32), HDIT_EPI_GATE_RESIDUAL only; may alias c
                        when both have one element type */
  const float* gate; /* f32, element (batch, col) at gate[batch * gate_stride + col] */
  int64_t lda, ldb, ldc, ldr;
  int32_t m, n, k;
  int32_t epilogue;
  int32_t rows_per_batch; /* rows of A per batch element (gate lookup) */
  int32_t gate_stride;
} hdit_gemm_problem;

int hdit_gemm_bf16(const hdit_gemm_problem* problems, int count, void* stream);

/* Test hook without a counterpart in the reference: pins the tile shape of
 * every later hdit_gemm_bf16 call of the process (0: 256x192, 1: 128x256,
 * 2: 128x128, 3: 256x256, 4: 128x192; -1: back to the planner). */
void hdit_gemm_force_config(int cfg);

/* ------------------------------------------------------------------------
 * Joint (image + text) flash attention, non-causal, no mask, bf16 in/out,
 * fp32 online softmax on MFMA.
 *
 * Q, K, V and O are each the concatenation, along the sequence, of up to two
 * segments that live in different buffers (segment 1 may have len 0): this is
 * the torch.cat([image, text]) of attention_processor.py:742-744 (SD3),
 * :894-896 (Flux, [text, image]) and the cat([text-K, cached image-K]) of
 * :908-922 without the copy.  Element (b, s, h, e) of a segment is at
 * ptr[b*stride_b + s*stride_s + h*stride_h + e]; head_dim is contiguous and
 * must be 64 or 128; strides must be multiples of 8 elements and pointers
 * 16-byte aligned.  sum(q.len) may differ from sum(k.len) (a PipeFusion query
 * patch against the whole stale K/V buffer); k and v segment lengths must
 * agree.  scale <= 0 selects 1/sqrt(head_dim), which is what the reference's
 * flash_attn_func / F.scaled_dot_product_attention calls use (:752-779,
 * :962-971, :1139-1151).
 * ---------------------------------------------------------------------- */
typedef struct hdit_seq_segment {
  const void* ptr;
  int64_t stride_b, stride_s, stride_h;
  int32_t len;
  int32_t pad_;
} hdit_seq_segment;

typedef struct hdit_attn_args {
  hdit_seq_segment q[2], k[2], v[2], o[2]; /* o[i].ptr is written */
  int32_t batch, heads, head_dim;
  float scale;
} hdit_attn_args;

int hdit_attn_fwd_bf16(const hdit_attn_args* args, void* stream);

/* `count` (<= HDIT_ATTN_MAX_MULTI) independent attention problems of one head dim
 * as ONE launch.  No single call site in the reference: the blocks (patch p, layer
 * l) with p + l constant of a PipeFusion step
 * (model_executor/pipelines/pipeline_stable_diffusion_3.py:1549-1644 runs them one
 * after the other) are independent, and each alone leaves most of the GPU idle.
 * Results are those of `count` hdit_attn_fwd_bf16 calls, bit for bit. */
#define HDIT_ATTN_MAX_MULTI 4
int hdit_attn_fwd_bf16_multi(const hdit_attn_args* args, int count, void* stream);

/* Same contract on the fp8-e4m3 (OCP) MFMA path: Q, K, V are quantised with one
 * absmax scale per (batch, head) taken from `absmax` (f32 [3, batch, heads]:
 * q, k, v; written by hdit_attn_absmax), P is re-quantised per tile.  K and V
 * are quantised once into `workspace` (hdit_attn_fp8_workspace_bytes(args)
 * bytes, 16-byte aligned, caller-owned).  No counterpart exists in the
 * reference (it has no fp8 path); the call site is that of
 * hdit_attn_fwd_bf16. */
int hdit_attn_absmax(const hdit_attn_args* args, float* absmax, void* stream);
int64_t hdit_attn_fp8_workspace_bytes(const hdit_attn_args* args);
int hdit_attn_fwd_fp8(const hdit_attn_args* args, const float* absmax, void* workspace, void* stream);

/* hdit_attn_fwd_fp8 without a workspace argument, for callers that cannot
 * allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * The quantised K / V copy goes into a fixed array inside the library's device
 * image (HDIT_ATTN_FP8_STATIC_MAX_BYTES per GPU, held until the process ends)
 * instead; the call allocates and frees nothing.  Results are bit-identical to
 * hdit_attn_fwd_fp8 on the same arguments.  A problem whose workspace
 * (hdit_attn_fp8_workspace_bytes) exceeds the array is refused with
 * HDIT_ETOOLARGE and a message in hdit_last_error.  All calls on one GPU share
 * that GPU's array: calls that overlap there (two streams, two threads) race;
 * serialise them.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress): make that call outside graph capture. */
#define HDIT_ATTN_FP8_STATIC_MAX_BYTES (32u << 20)
int hdit_attn_fwd_fp8_static(const hdit_attn_args* args, const float* absmax, void* stream);

/* ------------------------------------------------------------------------
 * Bandwidth-bound glue, one coalesced pass each.
 * ---------------------------------------------------------------------- */

/* y[b,t,:] = LayerNorm(x[b,t,:]; eps, optional affine ln_weight/ln_bias (bf16))
 *            * (1 + scale[b,:]) + shift[b,:]
 * x, y bf16 [batch, tokens, dim]: element (b, t, e) at ptr[b*_sb + t*_st + e]
 * (so a stream can be read from / written into a slice of a joint buffer);
 * shift/scale f32 with batch stride mod_stride (NULL => 0).
 * dim % 8 == 0, dim <= 8192.  Replaces diffusers AdaLayerNormZero /
 * AdaLayerNormZeroSingle / AdaLayerNormContinuous / CogVideoXLayerNormZero and
 * the norm2 + modulate of the blocks called at transformer_sd3.py:136-152,
 * transformer_flux.py:160-165,:194-198, cogvideox_transformer_3d.py:122-127. */
int hdit_layernorm_modulate(const void* x, void* y, const float* shift, const float* scale,
                            const void* ln_weight, const void* ln_bias, int batch, int tokens,
                            int dim, int64_t x_sb, int64_t x_st, int64_t y_sb, int64_t y_st,
                            int64_t mod_stride, float eps, void* stream);

/* The same for up to HDIT_LN_MAX_JOBS tensors of one width in one launch (the
 * image and the text stream of a joint block: norm1 + norm1_context, or
 * norm2 + norm2_context, of the blocks cited above). */
#define HDIT_LN_MAX_JOBS 8
typedef struct hdit_ln_job {
  const void* x;      /* bf16 [batch, tokens, dim], or f32 with x_f32 */
  void* y;            /* bf16 [batch, tokens, dim] */
  const float* shift; /* f32, batch stride mod_stride, or NULL */
  const float* scale;
  int64_t x_sb, x_st, y_sb, y_st, mod_stride;
  int32_t batch, tokens;
  int32_t x_f32; /* != 0: x is f32 [batch, tokens, dim] (strides in f32 elements): the fp32 residual stream */
  int32_t pad_;
  /* Optional pending update of the fp32 stream (x_f32 only; all NULL / 0 otherwise), applied before the
   * statistics: x' = x + delta_gate[b, :] * delta_y -- the gated residual `hidden_states + gate * attn_output`
   * (or `+ gate * ff_output`) of the blocks cited above, when the projection's GEMM wrote only
   * delta_y = bf16(A W^T + bias) and left the addition to the normalisation that reads the stream next.
   * delta_y bf16 [batch, tokens, dim] (strides d_sb, d_st), delta_gate f32 (batch stride gate_stride);
   * x_out != NULL: x' is written there as f32 (strides xo_sb, xo_st; may be x itself).  The result is
   * fma(gate, delta_y, x) per element, what HDIT_EPI_GATE_RESIDUAL computes. */
  const void* delta_y;
  const float* delta_gate;
  void* x_out;
  int64_t d_sb, d_st, gate_stride, xo_sb, xo_st;
} hdit_ln_job;

int hdit_layernorm_modulate_jobs(const hdit_ln_job* jobs, int count, int dim, const void* ln_weight,
                                 const void* ln_bias, float eps, void* stream);

/* out = x + gate[b,:] * y   (bf16 [batch, tokens, dim], gate f32).  The gated
 * residual of the same blocks when it is not fused into a GEMM epilogue. */
int hdit_gate_residual(const void* x, const void* y, const float* gate, void* out, int batch,
                       int tokens, int dim, int64_t x_sb, int64_t x_st, int64_t y_sb, int64_t y_st,
                       int64_t o_sb, int64_t o_st, int64_t gate_stride, void* stream);

/* out[b, :] = W . silu(temb[b, :]) + bias   (W bf16 [n, k], temb bf16 [batch, k],
 * bias bf16 [n] or NULL, out f32 [batch, n]); batch <= 8, k % 8 == 0, k <= 4096.
 * The `linear(silu(emb))` of every adaLN module (weight-bandwidth bound). */
int hdit_adaln_gemv(const void* temb, const void* w, const void* bias, float* out, int batch,
                    int n, int k, void* stream);

/* y = gelu_tanh(x + bias) elementwise (bf16 [rows, dim]); bias may be NULL.
 * diffusers GELU(approximate="tanh") inside the FeedForward wrapped at
 * layers/feedforward.py:17-78, when not fused into the GEMM epilogue. */
int hdit_gelu_tanh(const void* x, const void* bias, void* y, int64_t rows, int dim, int64_t ldx,
                   int64_t ldy, void* stream);

/* The feed-forward activations that have no fused GEMM epilogue, applied to the first projection's output
 * x [rows, ldx] (bias already added) -> y [rows, dim] (bf16):
 *   HDIT_ACT_GELU_ERF  y = gelu(x), exact          diffusers GELU(approximate="none")
 *   HDIT_ACT_GEGLU     y = x[:, :dim] * gelu(x[:, dim:2*dim])   diffusers GEGLU
 *   HDIT_ACT_SILU      y = silu(x)                 diffusers LinearActivation
 * the first-layer classes layers/feedforward.py:25-57 accepts besides the tanh GELU.  In place (y == x) except
 * for GEGLU. */
#define HDIT_ACT_GELU_ERF 0
#define HDIT_ACT_GEGLU 1
#define HDIT_ACT_SILU 2
int hdit_ff_activation(const void* x, void* y, int64_t rows, int dim, int64_t ldx, int64_t ldy, int kind,
                       void* stream);

/* In-place per-head QK normalisation + rotary embedding on x[b, s, h, :]
 * (bf16, strides as in hdit_seq_segment, head_dim 64 or 128):
 *   norm_kind 0: none; 1: RMSNorm(eps, weight); 2: LayerNorm(eps, weight, bias)
 *   then, for rows s in [rope_row0, rope_row0 + rope_rows):
 *   out = x*cos[s - rope_row0] + rotate_pairs(x)*sin[s - rope_row0]  (fp32 math)
 * cos/sin f32 [rope_rows, head_dim] (NULL => no rotation); rope_rows must cover
 * seq - rope_row0 rows (HDIT_EINVAL otherwise).  Up to 4 jobs per
 * launch.  Replaces attn.norm_q/norm_k/norm_added_q/norm_added_k and
 * apply_rotary_emb at attention_processor.py:68-120,:859-905,:1069-1082. */
typedef struct hdit_qknorm_job {
  void* x;
  int64_t stride_b, stride_s, stride_h;
  const void* weight; /* bf16 [head_dim] or NULL */
  const void* bias;   /* bf16 [head_dim] or NULL */
  const float* cos_table;
  const float* sin_table;
  int32_t seq, rope_row0, rope_rows, norm_kind;
} hdit_qknorm_job;

int hdit_qk_norm_rope(const hdit_qknorm_job* jobs, int count, int batch, int heads, int head_dim,
                      float eps, void* stream);

/* Plain strided copy of bf16 rows: dst[b, t, :dim] = src[b, t, :dim]; used to
 * place a [batch, tokens, dim] tensor into a slice of a larger buffer (the
 * in-place K/V patch overwrite of core/resource_manager/cache_manager.py:208-231).
 * dim % 8 == 0. */
int hdit_copy_rows(const void* src, void* dst, int batch, int tokens, int dim, int64_t src_sb,
                   int64_t src_st, int64_t dst_sb, int64_t dst_st, void* stream);

/* ------------------------------------------------------------------------
 * Head and tail of a denoise step around the block stack (about a megabyte
 * each; the projections between them are hdit_gemm_bf16 problems).
 * ---------------------------------------------------------------------- */

/* Rotary table from token positions: positions f32 [rows, n_axes]; per axis a
 * of width axes_dim[a] (even), angle = pos * theta^(-2i / axes_dim[a]) in float64,
 * each value written twice (rotation pair), axes concatenated: cos_out, sin_out
 * f32 [rows, sum(axes_dim)].  This is `self.pos_embed(ids)` of
 * models/transformers/transformer_flux.py:130-131 (axes (16, 56, 56) over
 * (0, row, col) ids) and the table the CogVideoX pipeline hands its blocks. */
#define HDIT_ROPE_MAX_AXES 4
int hdit_rope_table(const float* positions, int rows, const int* axes_dim, int n_axes, double theta, float* cos_out,
                    float* sin_out, void* stream);

/* out[b, hy*(W/p) + wx, (c*p + py)*p + px] = latent[b, c, hy*p + py, wx*p + px]
 * (bf16): the rows a p x p, stride-p convolution multiplies with its flattened
 * weight [out, c*p*p], i.e. the A operand that turns `self.module.proj(latent)`
 * + flatten + transpose of layers/embeddings.py:53-55 into a GEMM. */
int hdit_patchify(const void* latent, void* out, int batch, int channels, int height, int width, int patch,
                  void* stream);

/* out[b, c, hy*p + py, wx*p + px] = x[b, hy*(W/p) + wx, col] (bf16) with
 * col = (py*p + px)*C + c: the reshape + einsum("nhwpqc->nchpwq") + reshape of
 * models/transformers/transformer_sd3.py:160-182; or, channel_major != 0,
 * col = (c*p + py)*p + px: the reshape + permute(0, 1, 4, 2, 5, 3, 6) of
 * models/transformers/cogvideox_transformer_3d.py:143-146 with the frames of a
 * video counted into `batch`. */
int hdit_unpatchify(const void* x, void* out, int batch, int channels, int height, int width, int patch,
                    int channel_major, void* stream);

/* out[b, :dim/2] = cos(t[b] f_i), out[b, dim/2:] = sin(t[b] f_i), f_i =
 * max_period^(-i / (dim/2)); t f32 [batch], out bf16 [batch, dim].  diffusers
 * Timesteps(flip_sin_to_cos=True, downscale_freq_shift=0) inside the
 * time_text_embed called at transformer_sd3.py:101. */
int hdit_timestep_embedding(const float* timesteps, void* out, int batch, int dim, float max_period, void* stream);

/* y = silu(x) elementwise (bf16, count % 8 == 0): the activation between the
 * two linears of the timestep / pooled-text embedders of the same module. */
int hdit_silu(const void* x, void* y, int64_t count, void* stream);

/* Classifier-free guidance fused with the flow-match Euler update (bf16 in/out,
 * fp32 inside, in the rounding sequence of the tensor expressions replaced):
 *   noise = uncond + guidance * (cond - uncond)
 *     (model_executor/pipelines/pipeline_stable_diffusion_3.py:1703-1713)
 *   out = sample + ((sample - (sample - noise * sigma)) / sigma) * (sigma_next - sigma)
 *     (schedulers/scheduling_flow_match_euler_discrete.py:74-118 with gamma = 0) */
int hdit_cfg_euler_step(const void* noise_uncond, const void* noise_cond, const void* sample, void* out,
                        int64_t count, float guidance, float sigma, float sigma_next, void* stream);

/* ------------------------------------------------------------------------
 * One SD3 MMDiT joint block (diffusers JointTransformerBlock with the reference's
 * attention / feed-forward wrappers applied) as one call: adaLN projections,
 * norm1 + modulate, q|k|v of both streams, joint attention over [image, text],
 * out-projections with the gated residual, norm2 + modulate, GELU-tanh MLP with
 * the gated residual -- the launch sequence of the Python block, for hosts that
 * are not Python.  It is what the block loop of
 * models/transformers/transformer_sd3.py:107-152 calls per layer.
 *
 * All tensors are contiguous.  hidden [batch, n_img, dim], encoder [batch, n_txt,
 * dim] are bf16, or f32 with hidden_f32 / encoder_f32 (the residual stream of a
 * stack carried in fp32); temb bf16 [batch, temb_dim]; outputs bf16, or f32 with
 * out_f32.  Weights are bf16 nn.Linear weights [out, in] and biases [out] (NULL =
 * no bias): qkv_w = [to_q; to_k; to_v] packed [3 dim, dim], add_qkv_w likewise
 * for the text stream, norm1_w [6 dim, temb_dim], norm1_context_w [6 dim,
 * temb_dim] (context_pre_only: [2 dim, temb_dim], chunk order scale, shift).
 * context_pre_only != 0: last block -- no text out-projection, no text MLP,
 * encoder_out is not written.  skip_text_output != 0: the caller drops the text
 * output (pipeline patches after the first): the text stream only supplies keys
 * and values.  kv_buffer != NULL: the stale K|V buffer of a PipeFusion patch,
 * bf16 [batch, kv_rows, 2 dim] (k | v per row): this call's image rows overwrite
 * rows [kv_row0, kv_row0 + n_img) and attention reads all kv_rows
 * (core/resource_manager/cache_manager.py:117-149).  modulation_img /
 * modulation_txt: optional precomputed linear(silu(temb)) of norm1 /
 * norm1_context (f32 [batch, 6 dim] / [batch, 6 dim or 2 dim]); NULL => computed
 * here.  text_kv (optional): bf16 [batch, n_txt, 2 dim], the text stream's keys |
 * values.  text_kv_mode HDIT_TEXT_KV_STORE: this call projects them into that
 * buffer instead of the workspace.  HDIT_TEXT_KV_REUSE (only with
 * skip_text_output): the buffer already holds them -- models/transformers/
 * transformer_sd3.py:131-146 feeds every later patch of a step the text states
 * the first patch stored, so with the same temb their keys and values are the
 * numbers the first patch's call stored -- and the text stream's norm1 and
 * projection are not run.  fp8_attention != 0: the attention runs on the fp8-e4m3
 * path (hdit_attn_absmax + hdit_attn_fwd_fp8, their scales and quantised K / V
 * copy in the workspace).  workspace: hdit_block_sd3_workspace_bytes(args) bytes, 256-byte aligned,
 * caller-owned, contents undefined afterwards.
 * Arguments are validated before anything is enqueued.  A block is a sequence of
 * this library's launches, so if a later launch is refused (HDIT_ELAUNCH from the
 * runtime) the earlier ones are already on the stream and the outputs are
 * undefined; the return code is that launch's.
 * ---------------------------------------------------------------------- */
typedef struct hdit_sd3_block_weights {
  const void *norm1_w, *norm1_b, *norm1_context_w, *norm1_context_b;
  const void *qkv_w, *qkv_b, *add_qkv_w, *add_qkv_b;
  const void *to_out_w, *to_out_b, *to_add_out_w, *to_add_out_b;
  const void *ff_in_w, *ff_in_b, *ff_out_w, *ff_out_b;
  const void *ff_context_in_w, *ff_context_in_b, *ff_context_out_w, *ff_context_out_b;
} hdit_sd3_block_weights;

typedef struct hdit_sd3_block_args {
  hdit_sd3_block_weights w;
  const void* hidden;
  const void* encoder;
  const void* temb;
  void* hidden_out;
  void* encoder_out;
  const float* modulation_img;
  const float* modulation_txt;
  void* kv_buffer;
  void* workspace;
  int64_t workspace_bytes;
  int32_t batch, n_img, n_txt, dim, heads, ff_dim, temb_dim;
  int32_t kv_rows, kv_row0;
  int32_t hidden_f32, encoder_f32, out_f32;
  int32_t context_pre_only, skip_text_output;
  void* text_kv;
  int32_t text_kv_mode;
  int32_t fp8_attention;
  /* Gated residuals left to the next normalisation (fp32 streams only; all optional).
   * pending_img / pending_txt: bf16 [batch, n_img | n_txt, dim], an update still owed to `hidden` / `encoder`:
   * the stream this block works on is hidden + pending_img_gate[b, :] * pending_img (gate f32, batch stride
   * pending_*_gate_stride) -- applied inside norm1 / norm1_context.  defer_img / defer_txt (need out_f32 and
   * modulation_img / modulation_txt): the MLP's output projection writes bf16(A W^T + bias) there instead of
   * adding it; hidden_out / encoder_out then hold the stream after the attention residual, and the caller passes
   * (defer_*, modulation_* + 5 dim, 6 dim) as the next block's pending_*.  The sums are the ones the fused epilogue
   * makes, fma(gate, y, x) in fp32, so a stack run this way returns the same bits. */
  const void* pending_img;
  const float* pending_img_gate;
  const void* pending_txt;
  const float* pending_txt_gate;
  int64_t pending_img_gate_stride, pending_txt_gate_stride;
  void* defer_img;
  void* defer_txt;
  /* != 0: inside the block, too, the attention residual of a stream that arrives in f32 is added by norm2
   * (the out-projection writes bf16(A W^T + bias)) instead of in the out-projection's epilogue; same bits. */
  int32_t lazy_residual;
  int32_t pad_;
} hdit_sd3_block_args;

#define HDIT_TEXT_KV_NONE 0
#define HDIT_TEXT_KV_STORE 1
#define HDIT_TEXT_KV_REUSE 2

int64_t hdit_block_sd3_workspace_bytes(const hdit_sd3_block_args* args);
int hdit_block_sd3(const hdit_sd3_block_args* args, void* stream);

/* `count` (<= HDIT_BLOCK_MAX_MULTI) SD3 joint blocks that do not depend on each
 * other (one width and head count; each with its own workspace, K/V buffer and
 * outputs), run stage by stage with the launches of a stage merged: one
 * normalise launch, one grouped q|k|v GEMM, one attention launch
 * (hdit_attn_fwd_bf16_multi), ... for all of them.  These are the blocks (patch p,
 * layer l) with p + l constant of a PipeFusion step: the loop of
 * model_executor/pipelines/pipeline_stable_diffusion_3.py:1549-1644 runs patch after
 * patch through models/transformers/transformer_sd3.py:107-152, but block l of
 * patch p only needs block l of patch p - 1 and block l - 1 of its own patch, so
 * the blocks on a diagonal are independent, and a patch-sized launch alone fills
 * a fraction of the GPU.  Every output and K/V buffer is what `count`
 * hdit_block_sd3 calls in array order produce, bit for bit.  Everything is
 * validated before anything is enqueued. */
#define HDIT_BLOCK_MAX_MULTI 4
int hdit_block_sd3_multi(const hdit_sd3_block_args* args, int count, void* stream);

/* The Flux double-stream block (diffusers FluxTransformerBlock, called at
 * models/transformers/transformer_flux.py:160-165) as one call.  Weights as in
 * hdit_sd3_block_weights (every member present; to_add_out_b is ignored: the
 * reference's wrapper drops that bias in its Flux branch,
 * layers/attention_processor.py:176-192,:284-305) plus the per-head norm weights
 * of q, k of both streams (bf16 [head_dim] or NULL; qk_norm_kind as in
 * hdit_qknorm_job, qk_norm_eps its eps).  rope_cos / rope_sin: f32 [n_txt + n_img,
 * head_dim] over this call's joint [text, image] rows, or both NULL.
 * modulation_img / modulation_txt: optional precomputed linear(silu(temb)) of
 * norm1 / norm1_context (f32 [batch, 6 dim]); NULL => computed here.  kv_buffer !=
 * NULL: the image stream's K|V buffer of the layer, bf16 [batch, kv_rows, 2 dim]
 * (core/resource_manager/cache_manager.py:88-149, the call at
 * layers/attention_processor.py:908-922): this call projects its image rows' k | v
 * into rows [kv_row0, kv_row0 + n_img) (k normed and rotated there, in place) and
 * attention reads the text keys / values followed by all kv_rows -- a pipeline patch
 * over the stale rows of the other patches; batch <= HDIT_GEMM_MAX_PROBLEMS - 2
 * then.  Tensor conventions and workspace as for hdit_block_sd3. */
typedef struct hdit_flux_double_block_args {
  hdit_sd3_block_weights w;
  const void *norm_q_w, *norm_k_w, *norm_added_q_w, *norm_added_k_w;
  const void* hidden;
  const void* encoder;
  const void* temb;
  const float* rope_cos;
  const float* rope_sin;
  void* hidden_out;
  void* encoder_out;
  void* workspace;
  int64_t workspace_bytes;
  float qk_norm_eps;
  int32_t qk_norm_kind;
  int32_t batch, n_img, n_txt, dim, heads, ff_dim, temb_dim;
  int32_t hidden_f32, encoder_f32, out_f32;
  int32_t kv_rows, kv_row0;
  const float* modulation_img;
  const float* modulation_txt;
  void* kv_buffer;
} hdit_flux_double_block_args;

int64_t hdit_block_flux_double_workspace_bytes(const hdit_flux_double_block_args* args);
int hdit_block_flux_double(const hdit_flux_double_block_args* args, void* stream);

/* The Flux single-stream block (diffusers FluxSingleTransformerBlock,
 * transformer_flux.py:194-198) on the joint [text, image] sequence hidden
 * [batch, seq, dim]: adaLN-ZeroSingle (norm_w [3 dim, temb_dim]: shift, scale,
 * gate), q|k|v and proj_mlp in one launch, attention output and GELU(MLP) side by
 * side in one buffer, proj_out [dim, dim + ff_dim] with the gated residual.
 * modulation: optional precomputed linear(silu(temb)) (f32 [batch, 3 dim]).
 * kv_buffer != NULL (patch mode, layers/attention_processor.py:908-922): the first
 * n_txt rows of the sequence are text, the other seq - n_txt rows the image rows
 * of this pipeline patch; their k | v go into rows [kv_row0, kv_row0 + seq - n_txt)
 * of the layer's buffer bf16 [batch, kv_rows, 2 dim] and attention reads the text
 * keys / values followed by all kv_rows; 2 batch + 2 <= HDIT_GEMM_MAX_PROBLEMS. */
typedef struct hdit_flux_single_block_args {
  const void *norm_w, *norm_b, *qkv_w, *qkv_b, *proj_mlp_w, *proj_mlp_b, *proj_out_w, *proj_out_b, *norm_q_w, *norm_k_w;
  const void* hidden;
  const void* temb;
  const float* rope_cos;
  const float* rope_sin;
  void* hidden_out;
  void* workspace;
  int64_t workspace_bytes;
  float qk_norm_eps;
  int32_t qk_norm_kind;
  int32_t batch, seq, dim, heads, ff_dim, temb_dim;
  int32_t hidden_f32, out_f32;
  int32_t n_txt, kv_rows, kv_row0, pad_;
  const float* modulation;
  void* kv_buffer;
} hdit_flux_single_block_args;

int64_t hdit_block_flux_single_workspace_bytes(const hdit_flux_single_block_args* args);
int hdit_block_flux_single(const hdit_flux_single_block_args* args, void* stream);

/* The CogVideoX block (diffusers CogVideoXBlock, called at
 * models/transformers/cogvideox_transformer_3d.py:122-127): norm1_w / norm2_w
 * [6 dim, temb_dim] (shift, scale, gate, enc_shift, enc_scale, enc_gate),
 * norm*_ln_w / norm*_ln_b the affine LayerNorm [dim] shared by both streams
 * (norm_eps), one projection set over the joint [text, video] rows, LayerNorm or
 * RMSNorm per head on q, k (qk_norm_kind, weights / biases [head_dim]), rotation
 * of the video rows only (rope_cos / rope_sin f32 [n_img, head_dim] or NULL),
 * batch <= HDIT_GEMM_MAX_PROBLEMS / 2.  fp8_attention != 0: the attention on the
 * fp8-e4m3 path, as in hdit_block_sd3.  Returns hidden_out [batch, n_img, dim] and
 * encoder_out [batch, n_txt, dim]. */
typedef struct hdit_cogvideox_block_args {
  const void *norm1_w, *norm1_b, *norm1_ln_w, *norm1_ln_b, *norm2_w, *norm2_b, *norm2_ln_w, *norm2_ln_b;
  const void *qkv_w, *qkv_b, *to_out_w, *to_out_b, *norm_q_w, *norm_q_b, *norm_k_w, *norm_k_b;
  const void *ff_in_w, *ff_in_b, *ff_out_w, *ff_out_b;
  const void* hidden;
  const void* encoder;
  const void* temb;
  const float* rope_cos;
  const float* rope_sin;
  void* hidden_out;
  void* encoder_out;
  void* workspace;
  int64_t workspace_bytes;
  float norm_eps, qk_norm_eps;
  int32_t qk_norm_kind;
  int32_t batch, n_img, n_txt, dim, heads, ff_dim, temb_dim;
  int32_t hidden_f32, encoder_f32, out_f32;
  int32_t fp8_attention;
  const float* modulation1;  /* optional precomputed linear(silu(temb)) of norm1 / norm2, f32 [batch, 6 dim] */
  const float* modulation2;
} hdit_cogvideox_block_args;

int64_t hdit_block_cogvideox_workspace_bytes(const hdit_cogvideox_block_args* args);
int hdit_block_cogvideox(const hdit_cogvideox_block_args* args, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HDIT_H */
