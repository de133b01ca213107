// Whole-block entry points of the C ABI: the composition of the kernels that the Python blocks
// (hetu_dit_amd/blocks.py) make, for hosts that are not Python.  Pure host code: every step is one of the
// library's own entry points, enqueued on the caller's stream, with the intermediates in a caller workspace.
#include <string.h>

#include "hdit_common.h"

namespace {

constexpr int64_t ALIGN = 256;
int64_t up(int64_t x) { return (x + ALIGN - 1) / ALIGN * ALIGN; }

// Carves the workspace of one SD3 joint block; with base == nullptr it only measures.
struct Sd3Workspace {
  float* emb_img;   // [B, 6D]
  float* emb_txt;   // [B, 6D] (context_pre_only: [B, 2D])
  unsigned char* n_img;    // bf16 [B, Ni, D]: norm1 output, later norm2 output
  unsigned char* n_txt;    // bf16 [B, Nt, D]
  unsigned char* qkv_img;  // bf16 [B, Ni, 3D] (stale K/V buffer given: q only, [B, Ni, D])
  unsigned char* qkv_txt;  // bf16 [B, Nt, 3D] (text output skipped: k|v only, [B, Nt, 2D])
  unsigned char* o_img;    // bf16 [B, Ni, D]
  unsigned char* o_txt;    // bf16 [B, Nt, D]
  float* x1_img;           // f32 [B, Ni, D]: stream after the attention residual
  float* x1_txt;           // f32 [B, Nt, D]
  unsigned char* h_img;    // bf16 [B, Ni, F]
  unsigned char* h_txt;    // bf16 [B, Nt, F]
  float* absmax;           // f32 [3, B, H]: scales of the fp8 attention path
  unsigned char* fp8;      // its quantised K / V copy
  int64_t bytes;
};

// Workspace of the fp8 attention of this block: the size depends on the sequence lengths only, so the size query
// describes the segments with a placeholder address.
int64_t fp8_attention_bytes(const hdit_sd3_block_args* a) {
  const int hd = a->dim / a->heads;
  const int kv_rows = a->kv_buffer ? a->kv_rows : a->n_img;
  hdit_attn_args at;
  memset(&at, 0, sizeof(at));
  const void* somewhere = (const void*)(uintptr_t)256;
  auto seg = [&](hdit_seq_segment& s, int len) {
    s.ptr = somewhere, s.stride_b = (int64_t)len * a->dim, s.stride_s = a->dim, s.stride_h = hd, s.len = len;
  };
  seg(at.q[0], a->n_img), seg(at.o[0], a->n_img);
  seg(at.k[0], kv_rows), seg(at.v[0], kv_rows);
  seg(at.k[1], a->n_txt), seg(at.v[1], a->n_txt);
  if (!a->skip_text_output) seg(at.q[1], a->n_txt), seg(at.o[1], a->n_txt);
  at.batch = a->batch, at.heads = a->heads, at.head_dim = hd;
  return hdit_attn_fp8_workspace_bytes(&at);
}

Sd3Workspace carve(const hdit_sd3_block_args* a, unsigned char* base) {
  const int64_t B = a->batch, Ni = a->n_img, Nt = a->n_txt, D = a->dim, F = a->ff_dim;
  const bool text_out = !a->context_pre_only && !a->skip_text_output;
  Sd3Workspace w;
  int64_t off = 0;
  auto take = [&](int64_t nbytes) {
    unsigned char* p = base ? base + off : nullptr;
    off += up(nbytes);
    return p;
  };
  w.emb_img = (float*)take(B * 6 * D * 4);
  w.emb_txt = (float*)take(B * (a->context_pre_only ? 2 : 6) * D * 4);
  w.n_img = take(B * Ni * D * 2);
  w.n_txt = take(B * Nt * D * 2);
  w.qkv_img = take(B * Ni * (a->kv_buffer ? 1 : 3) * D * 2);
  // text q|k|v; with a text_kv buffer the keys | values live there and only the queries (if any) are here
  const int txt_cols = a->text_kv_mode != HDIT_TEXT_KV_NONE ? (a->skip_text_output ? 0 : 1) : (a->skip_text_output ? 2 : 3);
  w.qkv_txt = take(B * Nt * txt_cols * D * 2);
  w.o_img = take(B * Ni * D * 2);
  w.o_txt = take(a->skip_text_output ? 0 : B * Nt * D * 2);
  w.x1_img = (float*)take(B * Ni * D * 4);
  w.x1_txt = (float*)take(text_out ? B * Nt * D * 4 : 0);
  w.h_img = take(B * Ni * F * 2);
  w.h_txt = take(text_out ? B * Nt * F * 2 : 0);
  w.absmax = (float*)take(a->fp8_attention ? 3 * B * a->heads * 4 : 0);
  w.fp8 = take(a->fp8_attention ? fp8_attention_bytes(a) : 0);
  w.bytes = off;
  return w;
}

int validate(const hdit_sd3_block_args* a) {
  if (!a) return HDIT_EINVAL;
  if (a->batch <= 0 || a->n_img <= 0 || a->n_txt <= 0 || a->dim <= 0 || a->heads <= 0 || a->ff_dim <= 0) return HDIT_EINVAL;
  if (a->dim % a->heads) return HDIT_EINVAL;
  const int hd = a->dim / a->heads;
  if (hd != 64 && hd != 128) return HDIT_EUNSUPPORTED;
  if (a->dim % 64 || a->ff_dim % 64) return HDIT_EUNSUPPORTED;
  if (!a->hidden || !a->encoder || !a->temb || !a->hidden_out) return HDIT_EINVAL;
  const hdit_sd3_block_weights& w = a->w;
  if (!w.norm1_w || !w.norm1_b || !w.norm1_context_w || !w.norm1_context_b || !w.qkv_w || !w.add_qkv_w || !w.to_out_w ||
      !w.ff_in_w || !w.ff_out_w)
    return HDIT_EINVAL;
  const bool text_out = !a->context_pre_only && !a->skip_text_output;
  if (text_out && (!a->encoder_out || !w.to_add_out_w || !w.ff_context_in_w || !w.ff_context_out_w)) return HDIT_EINVAL;
  if (a->kv_buffer && (a->kv_rows < a->n_img || a->kv_row0 < 0 || a->kv_row0 + a->n_img > a->kv_rows)) return HDIT_EINVAL;
  if (a->text_kv_mode < HDIT_TEXT_KV_NONE || a->text_kv_mode > HDIT_TEXT_KV_REUSE) return HDIT_EINVAL;
  if (a->text_kv_mode != HDIT_TEXT_KV_NONE && (!a->text_kv || (((uintptr_t)a->text_kv) & 15))) return HDIT_EINVAL;
  if (a->text_kv_mode == HDIT_TEXT_KV_REUSE && !a->skip_text_output) return HDIT_EINVAL;
  if (a->fp8_attention != 0 && a->fp8_attention != 1) return HDIT_EINVAL;
  if (a->fp8_attention && fp8_attention_bytes(a) < 0) return HDIT_EINVAL;
  // updates owed to the fp32 streams, and the ones this block leaves to its successor
  if (a->pending_img && (!a->hidden_f32 || !a->pending_img_gate || (((uintptr_t)a->pending_img) & 15))) return HDIT_EINVAL;
  if (a->pending_txt && (!a->encoder_f32 || !a->pending_txt_gate || (((uintptr_t)a->pending_txt) & 15))) return HDIT_EINVAL;
  if (a->lazy_residual != 0 && a->lazy_residual != 1) return HDIT_EINVAL;
  if (a->defer_img && (!a->out_f32 || !a->modulation_img || (((uintptr_t)a->defer_img) & 15))) return HDIT_EINVAL;
  if (a->defer_txt && (!text_out || !a->out_f32 || !a->modulation_txt || (((uintptr_t)a->defer_txt) & 15)))
    return HDIT_EINVAL;
  return HDIT_OK;
}

hdit_gemm_problem problem(const void* x, int64_t lda, const void* w, const void* bias, void* c, int64_t ldc, int m, int n,
                          int k, int epilogue) {
  hdit_gemm_problem p;
  memset(&p, 0, sizeof(p));
  p.a = x, p.b = w, p.c = c, p.bias = bias;
  p.lda = lda, p.ldb = k, p.ldc = ldc;
  p.m = m, p.n = n, p.k = k;
  p.epilogue = epilogue;
  return p;
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int64_t hdit_block_sd3_workspace_bytes(const hdit_sd3_block_args* a) {
  if (validate(a) != HDIT_OK) return -1;
  return carve(a, nullptr).bytes;
}

namespace {

// The launches of one SD3 joint block, stage by stage: what hdit_block_sd3 enqueues in this order, and what
// hdit_block_sd3_multi merges stage-wise over several independent blocks.
struct Sd3Plan {
  const hdit_sd3_block_args* a;
  Sd3Workspace ws;
  bool gemv_img, gemv_txt;   // adaLN projections to compute here (no precomputed modulation given)
  hdit_ln_job ln1[2], ln2[2];
  int n_ln1, n_ln2;
  hdit_gemm_problem qkv[HDIT_GEMM_MAX_PROBLEMS], outp[2], ff1[2], ff2[2];
  int n_qkv, n_out, n_ff1, n_ff2;
  hdit_attn_args attn;
};

int plan_sd3(const hdit_sd3_block_args* a, Sd3Plan& pl) {
  int rc = validate(a);
  if (rc != HDIT_OK) return rc;
  if (!a->workspace || (((uintptr_t)a->workspace) & (ALIGN - 1))) return HDIT_EINVAL;
  pl.a = a;
  pl.ws = carve(a, (unsigned char*)a->workspace);
  const Sd3Workspace& ws = pl.ws;
  if (a->workspace_bytes < ws.bytes) return HDIT_EINVAL;
  const hdit_sd3_block_weights& w = a->w;
  const int B = a->batch, Ni = a->n_img, Nt = a->n_txt, D = a->dim, F = a->ff_dim, H = a->heads, hd = D / H;
  const bool pre_only = a->context_pre_only != 0;
  const bool text_out = !pre_only && !a->skip_text_output;
  const int64_t md = 6 * (int64_t)D;                 // batch stride of the image stream's modulation
  const int64_t mdt = (pre_only ? 2 : 6) * (int64_t)D;

  // 1. adaLN projections: linear(silu(temb)) for both streams (a caller that already holds them for this temb --
  //    the projections of all blocks of a stack fit one launch -- passes them in and skips this step)
  const float* emb_img = a->modulation_img;
  const float* emb_txt = a->modulation_txt;
  const bool reuse_text_kv = a->text_kv_mode == HDIT_TEXT_KV_REUSE;  // the text stream is not touched at all
  pl.gemv_img = !emb_img;
  pl.gemv_txt = !emb_txt && !reuse_text_kv;
  if (pl.gemv_img) emb_img = ws.emb_img;
  if (pl.gemv_txt) emb_txt = ws.emb_txt;
  // chunks: shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp; AdaLayerNormContinuous: scale, shift
  const float *sh_a = emb_img, *sc_a = emb_img + D, *g_a = emb_img + 2 * D, *sh_m = emb_img + 3 * D, *sc_m = emb_img + 4 * D,
              *g_m = emb_img + 5 * D;
  const float *c_sh_a = nullptr, *c_sc_a = nullptr, *c_g_a = nullptr, *c_sh_m = nullptr, *c_sc_m = nullptr, *c_g_m = nullptr;
  if (reuse_text_kv) {
    // no text-stream modulation needed
  } else if (pre_only) {
    c_sc_a = emb_txt, c_sh_a = emb_txt + D;
  } else {
    c_sh_a = emb_txt, c_sc_a = emb_txt + D, c_g_a = emb_txt + 2 * D, c_sh_m = emb_txt + 3 * D, c_sc_m = emb_txt + 4 * D,
    c_g_m = emb_txt + 5 * D;
  }

  // 2. norm1 + modulate, both streams in one launch
  hdit_ln_job* jobs = pl.ln1;
  memset(pl.ln1, 0, sizeof(pl.ln1));
  jobs[0].x = a->hidden, jobs[0].y = ws.n_img, jobs[0].shift = sh_a, jobs[0].scale = sc_a;
  jobs[0].x_sb = (int64_t)Ni * D, jobs[0].x_st = D, jobs[0].y_sb = (int64_t)Ni * D, jobs[0].y_st = D, jobs[0].mod_stride = md;
  jobs[0].batch = B, jobs[0].tokens = Ni, jobs[0].x_f32 = a->hidden_f32;
  jobs[1].x = a->encoder, jobs[1].y = ws.n_txt, jobs[1].shift = c_sh_a, jobs[1].scale = c_sc_a;
  jobs[1].x_sb = (int64_t)Nt * D, jobs[1].x_st = D, jobs[1].y_sb = (int64_t)Nt * D, jobs[1].y_st = D, jobs[1].mod_stride = mdt;
  jobs[1].batch = B, jobs[1].tokens = Nt, jobs[1].x_f32 = a->encoder_f32;
  pl.n_ln1 = reuse_text_kv ? 1 : 2;
  // The fp32 streams inside the block.  A stream that arrives in fp32 takes its gated residuals in the
  // normalisation that reads it next (hdit_ln_job.delta_y) instead of in the projection's epilogue: the out-projection
  // and, with defer_img / defer_txt, the MLP's second projection write only bf16(A W^T + bias).  `st_*` is where the
  // updated stream lives: the block's output when the MLP's residual is left to the next block (the output is then
  // the stream after the attention residual), the workspace otherwise.
  const bool lazy_img = a->lazy_residual && a->hidden_f32 != 0, lazy_txt = a->lazy_residual && a->encoder_f32 != 0 && text_out;
  float* st_img = a->defer_img ? (float*)a->hidden_out : ws.x1_img;
  float* st_txt = a->defer_txt ? (float*)a->encoder_out : ws.x1_txt;
  const void* x0_img = a->hidden;
  const void* x0_txt = a->encoder;
  if (a->pending_img) {
    jobs[0].delta_y = a->pending_img, jobs[0].delta_gate = a->pending_img_gate, jobs[0].gate_stride = a->pending_img_gate_stride;
    jobs[0].d_sb = (int64_t)Ni * D, jobs[0].d_st = D;
    jobs[0].x_out = st_img, jobs[0].xo_sb = (int64_t)Ni * D, jobs[0].xo_st = D;
    x0_img = st_img;
  }
  if (a->pending_txt && !reuse_text_kv) {
    jobs[1].delta_y = a->pending_txt, jobs[1].delta_gate = a->pending_txt_gate, jobs[1].gate_stride = a->pending_txt_gate_stride;
    jobs[1].d_sb = (int64_t)Nt * D, jobs[1].d_st = D;
    if (text_out) {  // a stream without an output (context_pre_only, patches after the first) is only normalised
      jobs[1].x_out = st_txt, jobs[1].xo_sb = (int64_t)Nt * D, jobs[1].xo_st = D;
      x0_txt = st_txt;
    }
  }

  // 3. q|k|v of both streams in one grouped launch.  With a stale K/V buffer the image stream's k|v rows go
  //    straight into rows [kv_row0, kv_row0 + n_img) of it, one problem per batch element.
  hdit_gemm_problem* probs = pl.qkv;
  int np = 0;
  const unsigned char* qkv_w = (const unsigned char*)w.qkv_w;
  const unsigned char* qkv_b = (const unsigned char*)w.qkv_b;
  const unsigned char* aqkv_w = (const unsigned char*)w.add_qkv_w;
  const unsigned char* aqkv_b = (const unsigned char*)w.add_qkv_b;
  int64_t q_ld, kv_ld;         // row strides (elements) of the image q and k|v
  const unsigned char *q_img, *k_img, *v_img;
  int kv_img_rows;
  if (!a->kv_buffer) {
    probs[np++] = problem(ws.n_img, D, qkv_w, qkv_b, ws.qkv_img, 3 * D, B * Ni, 3 * D, D, HDIT_EPI_BIAS);
    q_ld = kv_ld = 3 * (int64_t)D;
    q_img = ws.qkv_img, k_img = ws.qkv_img + (int64_t)D * 2, v_img = ws.qkv_img + (int64_t)2 * D * 2;
    kv_img_rows = Ni;
  } else {
    if (B + 2 > HDIT_GEMM_MAX_PROBLEMS) return HDIT_EUNSUPPORTED;
    probs[np++] = problem(ws.n_img, D, qkv_w, qkv_b, ws.qkv_img, D, B * Ni, D, D, HDIT_EPI_BIAS);
    unsigned char* kvb = (unsigned char*)a->kv_buffer;
    for (int b = 0; b < B; b++)
      probs[np++] = problem(ws.n_img + (int64_t)b * Ni * D * 2, D, qkv_w + (int64_t)D * D * 2, qkv_b ? qkv_b + (int64_t)D * 2 : nullptr,
                            kvb + ((int64_t)b * a->kv_rows + a->kv_row0) * 2 * D * 2, 2 * D, Ni, 2 * D, D, HDIT_EPI_BIAS);
    q_ld = D, kv_ld = 2 * (int64_t)D;
    q_img = ws.qkv_img, k_img = kvb, v_img = kvb + (int64_t)D * 2;
    kv_img_rows = a->kv_rows;
  }
  int64_t tq_ld = 0, tkv_ld;  // row strides (elements) of the text q and k|v
  const unsigned char *q_txt = nullptr, *k_txt, *v_txt;
  if (a->text_kv_mode != HDIT_TEXT_KV_NONE) {
    if (np + 2 > HDIT_GEMM_MAX_PROBLEMS) return HDIT_EUNSUPPORTED;
    unsigned char* tkv = (unsigned char*)a->text_kv;
    if (!reuse_text_kv) {
      if (!a->skip_text_output) {
        probs[np++] = problem(ws.n_txt, D, aqkv_w, aqkv_b, ws.qkv_txt, D, B * Nt, D, D, HDIT_EPI_BIAS);
        q_txt = ws.qkv_txt, tq_ld = D;
      }
      probs[np++] = problem(ws.n_txt, D, aqkv_w + (int64_t)D * D * 2, aqkv_b ? aqkv_b + (int64_t)D * 2 : nullptr, tkv, 2 * D,
                            B * Nt, 2 * D, D, HDIT_EPI_BIAS);
    }
    tkv_ld = 2 * (int64_t)D;
    k_txt = tkv, v_txt = tkv + (int64_t)D * 2;
  } else if (a->skip_text_output) {
    probs[np++] = problem(ws.n_txt, D, aqkv_w + (int64_t)D * D * 2, aqkv_b ? aqkv_b + (int64_t)D * 2 : nullptr, ws.qkv_txt,
                          2 * D, B * Nt, 2 * D, D, HDIT_EPI_BIAS);
    tkv_ld = 2 * (int64_t)D;
    k_txt = ws.qkv_txt, v_txt = ws.qkv_txt + (int64_t)D * 2;
  } else {
    probs[np++] = problem(ws.n_txt, D, aqkv_w, aqkv_b, ws.qkv_txt, 3 * D, B * Nt, 3 * D, D, HDIT_EPI_BIAS);
    tq_ld = tkv_ld = 3 * (int64_t)D;
    q_txt = ws.qkv_txt, k_txt = ws.qkv_txt + (int64_t)D * 2, v_txt = ws.qkv_txt + (int64_t)2 * D * 2;
  }
  pl.n_qkv = np;

  // 4. joint attention over [image, text]; image keys / values come from the stale buffer when there is one
  hdit_attn_args& at = pl.attn;
  memset(&at, 0, sizeof(at));
  auto seg = [&](hdit_seq_segment& s, const void* p, int64_t rows_per_batch, int64_t ld, int len) {
    s.ptr = p, s.stride_b = rows_per_batch * ld, s.stride_s = ld, s.stride_h = hd, s.len = len;
  };
  seg(at.q[0], q_img, Ni, q_ld, Ni);
  seg(at.k[0], k_img, kv_img_rows, kv_ld, kv_img_rows);
  seg(at.v[0], v_img, kv_img_rows, kv_ld, kv_img_rows);
  seg(at.k[1], k_txt, Nt, tkv_ld, Nt);
  seg(at.v[1], v_txt, Nt, tkv_ld, Nt);
  seg(at.o[0], ws.o_img, Ni, D, Ni);
  if (!a->skip_text_output) {
    seg(at.q[1], q_txt, Nt, tq_ld, Nt);
    seg(at.o[1], ws.o_txt, Nt, D, Nt);
  }
  at.batch = B, at.heads = H, at.head_dim = hd, at.scale = 0.f;

  // 5. out-projections with the gated residual; the stream stays fp32 inside the block
  auto gated = [&](hdit_gemm_problem& p, const void* resid, int resid_f32, const float* gate, int64_t gate_stride, int rows,
                   int out_f32) {
    p.epilogue = HDIT_EPI_GATE_RESIDUAL | (resid_f32 ? HDIT_EPI_RESID_F32 : 0) | (out_f32 ? HDIT_EPI_OUT_F32 : 0);
    p.resid = resid, p.ldr = p.n, p.gate = gate, p.gate_stride = (int32_t)gate_stride, p.rows_per_batch = rows;
  };
  np = 0;
  // the projected attention output of a lazily updated stream goes where that stream's q (|k|v) was: dead since the attention
  if (lazy_img) {
    pl.outp[np++] = problem(ws.o_img, D, w.to_out_w, w.to_out_b, ws.qkv_img, D, B * Ni, D, D, HDIT_EPI_BIAS);
  } else {
    pl.outp[np] = problem(ws.o_img, D, w.to_out_w, w.to_out_b, st_img, D, B * Ni, D, D, 0);
    gated(pl.outp[np++], a->hidden, a->hidden_f32, g_a, md, Ni, 1);
  }
  if (text_out) {
    if (lazy_txt) {
      pl.outp[np++] = problem(ws.o_txt, D, w.to_add_out_w, w.to_add_out_b, ws.qkv_txt, D, B * Nt, D, D, HDIT_EPI_BIAS);
    } else {
      pl.outp[np] = problem(ws.o_txt, D, w.to_add_out_w, w.to_add_out_b, st_txt, D, B * Nt, D, D, 0);
      gated(pl.outp[np++], a->encoder, a->encoder_f32, c_g_a, mdt, Nt, 1);
    }
  }
  pl.n_out = np;

  // 6. norm2 + modulate on the fp32 stream
  int nj = 0;
  jobs = pl.ln2;
  memset(pl.ln2, 0, sizeof(pl.ln2));
  jobs[nj].x = lazy_img ? x0_img : st_img, jobs[nj].y = ws.n_img, jobs[nj].shift = sh_m, jobs[nj].scale = sc_m;
  jobs[nj].x_sb = (int64_t)Ni * D, jobs[nj].x_st = D, jobs[nj].y_sb = (int64_t)Ni * D, jobs[nj].y_st = D, jobs[nj].mod_stride = md;
  jobs[nj].batch = B, jobs[nj].tokens = Ni, jobs[nj].x_f32 = 1;
  if (lazy_img) {
    jobs[nj].delta_y = ws.qkv_img, jobs[nj].delta_gate = g_a, jobs[nj].gate_stride = md;
    jobs[nj].d_sb = (int64_t)Ni * D, jobs[nj].d_st = D;
    jobs[nj].x_out = st_img, jobs[nj].xo_sb = (int64_t)Ni * D, jobs[nj].xo_st = D;
  }
  nj++;
  if (text_out) {
    jobs[nj].x = lazy_txt ? x0_txt : st_txt, jobs[nj].y = ws.n_txt, jobs[nj].shift = c_sh_m, jobs[nj].scale = c_sc_m;
    jobs[nj].x_sb = (int64_t)Nt * D, jobs[nj].x_st = D, jobs[nj].y_sb = (int64_t)Nt * D, jobs[nj].y_st = D, jobs[nj].mod_stride = mdt;
    jobs[nj].batch = B, jobs[nj].tokens = Nt, jobs[nj].x_f32 = 1;
    if (lazy_txt) {
      jobs[nj].delta_y = ws.qkv_txt, jobs[nj].delta_gate = c_g_a, jobs[nj].gate_stride = mdt;
      jobs[nj].d_sb = (int64_t)Nt * D, jobs[nj].d_st = D;
      jobs[nj].x_out = st_txt, jobs[nj].xo_sb = (int64_t)Nt * D, jobs[nj].xo_st = D;
    }
    nj++;
  }
  pl.n_ln2 = nj;

  // 7. MLP: bias + GELU-tanh in the first epilogue, gated residual in the second
  np = 0;
  pl.ff1[np++] = problem(ws.n_img, D, w.ff_in_w, w.ff_in_b, ws.h_img, F, B * Ni, F, D, HDIT_EPI_BIAS_GELU);
  if (text_out) pl.ff1[np++] = problem(ws.n_txt, D, w.ff_context_in_w, w.ff_context_in_b, ws.h_txt, F, B * Nt, F, D, HDIT_EPI_BIAS_GELU);
  pl.n_ff1 = np;
  np = 0;
  if (a->defer_img) {
    pl.ff2[np++] = problem(ws.h_img, F, w.ff_out_w, w.ff_out_b, a->defer_img, D, B * Ni, D, F, HDIT_EPI_BIAS);
  } else {
    pl.ff2[np] = problem(ws.h_img, F, w.ff_out_w, w.ff_out_b, a->hidden_out, D, B * Ni, D, F, 0);
    gated(pl.ff2[np++], st_img, 1, g_m, md, Ni, a->out_f32);
  }
  if (text_out) {
    if (a->defer_txt) {
      pl.ff2[np++] = problem(ws.h_txt, F, w.ff_context_out_w, w.ff_context_out_b, a->defer_txt, D, B * Nt, D, F, HDIT_EPI_BIAS);
    } else {
      pl.ff2[np] = problem(ws.h_txt, F, w.ff_context_out_w, w.ff_context_out_b, a->encoder_out, D, B * Nt, D, F, 0);
      gated(pl.ff2[np++], st_txt, 1, c_g_m, mdt, Nt, a->out_f32);
    }
  }
  pl.n_ff2 = np;
  return HDIT_OK;
}

int run_gemvs(const Sd3Plan& pl, void* stream) {
  const hdit_sd3_block_args* a = pl.a;
  int rc;
  if (pl.gemv_img && (rc = hdit_adaln_gemv(a->temb, a->w.norm1_w, a->w.norm1_b, pl.ws.emb_img, a->batch, 6 * a->dim, a->temb_dim, stream)))
    return rc;
  if (pl.gemv_txt && (rc = hdit_adaln_gemv(a->temb, a->w.norm1_context_w, a->w.norm1_context_b, pl.ws.emb_txt, a->batch,
                                           (a->context_pre_only ? 2 : 6) * a->dim, a->temb_dim, stream)))
    return rc;
  return HDIT_OK;
}

int run_attention(const Sd3Plan& pl, void* stream) {
  int rc;
  if (pl.a->fp8_attention) {
    if ((rc = hdit_attn_absmax(&pl.attn, pl.ws.absmax, stream))) return rc;
    return hdit_attn_fwd_fp8(&pl.attn, pl.ws.absmax, pl.ws.fp8, stream);
  }
  return hdit_attn_fwd_bf16(&pl.attn, stream);
}

// Problems of several plans, one launch per HDIT_GEMM_MAX_PROBLEMS (a launch plans its problems together).
template <class Get>
int run_gemm_stage(const Sd3Plan* plans, int count, Get get, void* stream) {
  hdit_gemm_problem probs[HDIT_GEMM_MAX_PROBLEMS];
  int np = 0, rc;
  for (int i = 0; i < count; i++) {
    int n;
    const hdit_gemm_problem* p = get(plans[i], n);
    if (np + n > HDIT_GEMM_MAX_PROBLEMS) {
      if ((rc = hdit_gemm_bf16(probs, np, stream))) return rc;
      np = 0;
    }
    for (int k = 0; k < n; k++) probs[np++] = p[k];
  }
  return np ? hdit_gemm_bf16(probs, np, stream) : HDIT_OK;
}

template <class Get>
int run_ln_stage(const Sd3Plan* plans, int count, Get get, int dim, void* stream) {
  hdit_ln_job jobs[HDIT_LN_MAX_JOBS];
  int nj = 0, rc;
  for (int i = 0; i < count; i++) {
    int n;
    const hdit_ln_job* j = get(plans[i], n);
    if (nj + n > HDIT_LN_MAX_JOBS) {
      if ((rc = hdit_layernorm_modulate_jobs(jobs, nj, dim, nullptr, nullptr, 1e-6f, stream))) return rc;
      nj = 0;
    }
    for (int k = 0; k < n; k++) jobs[nj++] = j[k];
  }
  return nj ? hdit_layernorm_modulate_jobs(jobs, nj, dim, nullptr, nullptr, 1e-6f, stream) : HDIT_OK;
}

// `count` planned blocks, stage by stage: the launches of each stage merged into one
int run_sd3_plans(const Sd3Plan* plans, int count, void* stream) {
  int rc;
  const int D = plans[0].a->dim;
  for (int i = 0; i < count; i++)
    if ((rc = run_gemvs(plans[i], stream))) return rc;
  if ((rc = run_ln_stage(plans, count, [](const Sd3Plan& p, int& n) { n = p.n_ln1; return p.ln1; }, D, stream))) return rc;
  if ((rc = run_gemm_stage(plans, count, [](const Sd3Plan& p, int& n) { n = p.n_qkv; return p.qkv; }, stream))) return rc;
  bool any_fp8 = false;
  for (int i = 0; i < count; i++) any_fp8 |= plans[i].a->fp8_attention != 0;
  if (count == 1 || any_fp8) {
    for (int i = 0; i < count; i++)
      if ((rc = run_attention(plans[i], stream))) return rc;
  } else {
    hdit_attn_args at[HDIT_ATTN_MAX_MULTI];
    for (int first = 0; first < count; first += HDIT_ATTN_MAX_MULTI) {
      const int n = count - first < HDIT_ATTN_MAX_MULTI ? count - first : HDIT_ATTN_MAX_MULTI;
      for (int i = 0; i < n; i++) at[i] = plans[first + i].attn;
      if ((rc = hdit_attn_fwd_bf16_multi(at, n, stream))) return rc;
    }
  }
  if ((rc = run_gemm_stage(plans, count, [](const Sd3Plan& p, int& n) { n = p.n_out; return p.outp; }, stream))) return rc;
  if ((rc = run_ln_stage(plans, count, [](const Sd3Plan& p, int& n) { n = p.n_ln2; return p.ln2; }, D, stream))) return rc;
  if ((rc = run_gemm_stage(plans, count, [](const Sd3Plan& p, int& n) { n = p.n_ff1; return p.ff1; }, stream))) return rc;
  return run_gemm_stage(plans, count, [](const Sd3Plan& p, int& n) { n = p.n_ff2; return p.ff2; }, stream);
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int hdit_block_sd3(const hdit_sd3_block_args* a, void* stream) {
  Sd3Plan pl;
  const int rc = plan_sd3(a, pl);
  if (rc != HDIT_OK) return rc;
  return run_sd3_plans(&pl, 1, stream);
}

extern "C" __attribute__((visibility("default"))) int hdit_block_sd3_multi(const hdit_sd3_block_args* args, int count, void* stream) {
  if (!args || count <= 0 || count > HDIT_BLOCK_MAX_MULTI) return HDIT_EINVAL;
  static thread_local Sd3Plan plans[HDIT_BLOCK_MAX_MULTI];
  for (int i = 0; i < count; i++) {
    const int rc = plan_sd3(&args[i], plans[i]);
    if (rc != HDIT_OK) return rc;
    if (args[i].dim != args[0].dim || args[i].heads != args[0].heads) return HDIT_EINVAL;
  }
  return run_sd3_plans(plans, count, stream);
}

// ---------------------------------------------------------------------------------------------------------
// Flux and CogVideoX blocks
// ---------------------------------------------------------------------------------------------------------
namespace {

struct Carver {
  unsigned char* base;
  int64_t off = 0;
  explicit Carver(void* b) : base((unsigned char*)b) {}
  unsigned char* take(int64_t nbytes) {
    unsigned char* p = base ? base + off : nullptr;
    off += up(nbytes);
    return p;
  }
};

void ln_job(hdit_ln_job& j, const void* x, int x_f32, void* y, int64_t y_sb, const float* shift, const float* scale,
            int64_t mod_stride, int batch, int tokens, int dim) {
  memset(&j, 0, sizeof(j));
  j.x = x, j.y = y, j.shift = shift, j.scale = scale;
  j.x_sb = (int64_t)tokens * dim, j.x_st = dim, j.y_sb = y_sb, j.y_st = dim, j.mod_stride = mod_stride;
  j.batch = batch, j.tokens = tokens, j.x_f32 = x_f32;
}

void gated(hdit_gemm_problem& p, const void* resid, int resid_f32, const float* gate, int64_t gate_stride, int rows,
           int out_f32) {
  p.epilogue = HDIT_EPI_GATE_RESIDUAL | (resid_f32 ? HDIT_EPI_RESID_F32 : 0) | (out_f32 ? HDIT_EPI_OUT_F32 : 0);
  p.resid = resid, p.ldr = p.n, p.gate = gate, p.gate_stride = (int32_t)gate_stride, p.rows_per_batch = rows;
}

void qk_job(hdit_qknorm_job& j, void* x, int64_t rows_per_batch, int64_t ld, int hd, const void* weight, const void* bias,
            const float* cos_t, const float* sin_t, int seq, int rope_row0, int rope_rows, int norm_kind) {
  memset(&j, 0, sizeof(j));
  j.x = x, j.stride_b = rows_per_batch * ld, j.stride_s = ld, j.stride_h = hd;
  j.weight = weight, j.bias = bias, j.cos_table = cos_t, j.sin_table = sin_t;
  j.seq = seq, j.rope_row0 = rope_row0, j.rope_rows = rope_rows, j.norm_kind = norm_kind;
}

void seg(hdit_seq_segment& s, const void* p, int64_t rows_per_batch, int64_t ld, int hd, int len) {
  s.ptr = p, s.stride_b = rows_per_batch * ld, s.stride_s = ld, s.stride_h = hd, s.len = len;
}

bool head_dim_ok(int dim, int heads) { return heads > 0 && dim % heads == 0 && (dim / heads == 64 || dim / heads == 128); }

struct FluxDoubleWs {
  float *emb_img, *emb_txt, *x1_img, *x1_txt;
  unsigned char *n_img, *n_txt, *qkv_img, *qkv_txt, *o_img, *o_txt, *h_img, *h_txt;
  int64_t bytes;
};
FluxDoubleWs carve(const hdit_flux_double_block_args* a, void* base) {
  const int64_t B = a->batch, Ni = a->n_img, Nt = a->n_txt, D = a->dim, F = a->ff_dim;
  Carver c(base);
  FluxDoubleWs w;
  w.emb_img = (float*)c.take(B * 6 * D * 4), w.emb_txt = (float*)c.take(B * 6 * D * 4);
  w.n_img = c.take(B * Ni * D * 2), w.n_txt = c.take(B * Nt * D * 2);
  w.qkv_img = c.take(B * Ni * (a->kv_buffer ? 1 : 3) * D * 2), w.qkv_txt = c.take(B * Nt * 3 * D * 2);  // buffer given: q only
  w.o_img = c.take(B * Ni * D * 2), w.o_txt = c.take(B * Nt * D * 2);
  w.x1_img = (float*)c.take(B * Ni * D * 4), w.x1_txt = (float*)c.take(B * Nt * D * 4);
  w.h_img = c.take(B * Ni * F * 2), w.h_txt = c.take(B * Nt * F * 2);
  w.bytes = c.off;
  return w;
}
int validate(const hdit_flux_double_block_args* a) {
  if (!a || a->batch <= 0 || a->n_img <= 0 || a->n_txt <= 0 || a->dim <= 0 || a->ff_dim <= 0 || a->temb_dim <= 0) return HDIT_EINVAL;
  if (!head_dim_ok(a->dim, a->heads)) return HDIT_EUNSUPPORTED;
  if (a->dim % 64 || a->ff_dim % 64) return HDIT_EUNSUPPORTED;
  const hdit_sd3_block_weights& w = a->w;
  if (!a->hidden || !a->encoder || !a->temb || !a->hidden_out || !a->encoder_out) return HDIT_EINVAL;
  if (!w.norm1_w || !w.norm1_b || !w.norm1_context_w || !w.norm1_context_b || !w.qkv_w || !w.add_qkv_w || !w.to_out_w ||
      !w.to_add_out_w || !w.ff_in_w || !w.ff_out_w || !w.ff_context_in_w || !w.ff_context_out_w)
    return HDIT_EINVAL;
  if ((a->rope_cos == nullptr) != (a->rope_sin == nullptr)) return HDIT_EINVAL;
  if (a->kv_buffer) {
    if ((((uintptr_t)a->kv_buffer) & 15) || a->kv_rows < a->n_img || a->kv_row0 < 0 || a->kv_row0 + a->n_img > a->kv_rows)
      return HDIT_EINVAL;
    if (a->batch + 2 > HDIT_GEMM_MAX_PROBLEMS) return HDIT_EUNSUPPORTED;
  }
  return HDIT_OK;
}

struct FluxSingleWs {
  float* emb;
  unsigned char *n, *qkv, *kv_txt, *cat;
  int64_t bytes;
};
FluxSingleWs carve(const hdit_flux_single_block_args* a, void* base) {
  const int64_t B = a->batch, S = a->seq, D = a->dim, F = a->ff_dim;
  Carver c(base);
  FluxSingleWs w;
  w.emb = (float*)c.take(B * 3 * D * 4);
  w.n = c.take(B * S * D * 2);
  // buffer given: q of all rows [B, S, D], then the text rows' k | v [B, n_txt, 2 D]
  w.qkv = c.take(a->kv_buffer ? B * S * D * 2 : B * S * 3 * D * 2);
  w.kv_txt = c.take(a->kv_buffer ? B * (int64_t)a->n_txt * 2 * D * 2 : 0);
  w.cat = c.take(B * S * (D + F) * 2);
  w.bytes = c.off;
  return w;
}
int validate(const hdit_flux_single_block_args* a) {
  if (!a || a->batch <= 0 || a->seq <= 0 || a->dim <= 0 || a->ff_dim <= 0 || a->temb_dim <= 0) return HDIT_EINVAL;
  if (!head_dim_ok(a->dim, a->heads)) return HDIT_EUNSUPPORTED;
  if (a->dim % 64 || a->ff_dim % 64) return HDIT_EUNSUPPORTED;
  if (!a->hidden || !a->temb || !a->hidden_out || !a->norm_w || !a->norm_b || !a->qkv_w || !a->proj_mlp_w || !a->proj_out_w)
    return HDIT_EINVAL;
  if ((a->rope_cos == nullptr) != (a->rope_sin == nullptr)) return HDIT_EINVAL;
  if (a->kv_buffer) {
    const int n_img = a->seq - a->n_txt;
    if ((((uintptr_t)a->kv_buffer) & 15) || a->n_txt < 0 || n_img <= 0) return HDIT_EINVAL;
    if (a->kv_rows < n_img || a->kv_row0 < 0 || a->kv_row0 + n_img > a->kv_rows) return HDIT_EINVAL;
    if (2 * a->batch + 2 > HDIT_GEMM_MAX_PROBLEMS) return HDIT_EUNSUPPORTED;
  }
  return HDIT_OK;
}

struct CogWs {
  float *emb1, *emb2, *x1_h, *x1_e, *absmax;
  unsigned char *joint, *qkv, *o, *h, *fp8;
  int64_t bytes;
};
// one joint [text, video] segment per tensor, q | k | v as column ranges of the packed projection
void cog_attn_args(const hdit_cogvideox_block_args* a, hdit_attn_args& at, const void* q, const void* k, const void* v,
                   void* o) {
  const int S = a->n_img + a->n_txt, D = a->dim, hd = D / a->heads;
  memset(&at, 0, sizeof(at));
  seg(at.q[0], q, S, 3 * (int64_t)D, hd, S), seg(at.k[0], k, S, 3 * (int64_t)D, hd, S), seg(at.v[0], v, S, 3 * (int64_t)D, hd, S);
  seg(at.o[0], o, S, D, hd, S);
  at.batch = a->batch, at.heads = a->heads, at.head_dim = hd, at.scale = 0.f;
}
int64_t cog_fp8_bytes(const hdit_cogvideox_block_args* a) {
  hdit_attn_args at;
  void* somewhere = (void*)(uintptr_t)256;  // the size depends on the lengths only
  cog_attn_args(a, at, somewhere, somewhere, somewhere, somewhere);
  return hdit_attn_fp8_workspace_bytes(&at);
}
CogWs carve(const hdit_cogvideox_block_args* a, void* base) {
  const int64_t B = a->batch, S = (int64_t)a->n_img + a->n_txt, D = a->dim, F = a->ff_dim;
  Carver c(base);
  CogWs w;
  w.emb1 = (float*)c.take(B * 6 * D * 4), w.emb2 = (float*)c.take(B * 6 * D * 4);
  w.joint = c.take(B * S * D * 2);
  w.qkv = c.take(B * S * 3 * D * 2);
  w.o = c.take(B * S * D * 2);
  w.x1_h = (float*)c.take(B * a->n_img * D * 4), w.x1_e = (float*)c.take(B * a->n_txt * D * 4);
  w.h = c.take(B * S * F * 2);
  w.absmax = (float*)c.take(a->fp8_attention ? 3 * B * a->heads * 4 : 0);
  w.fp8 = c.take(a->fp8_attention ? cog_fp8_bytes(a) : 0);
  w.bytes = c.off;
  return w;
}
int validate(const hdit_cogvideox_block_args* a) {
  if (!a || a->batch <= 0 || a->n_img <= 0 || a->n_txt <= 0 || a->dim <= 0 || a->ff_dim <= 0 || a->temb_dim <= 0) return HDIT_EINVAL;
  if (2 * a->batch > HDIT_GEMM_MAX_PROBLEMS) return HDIT_EUNSUPPORTED;
  if (!head_dim_ok(a->dim, a->heads)) return HDIT_EUNSUPPORTED;
  if (a->dim % 64 || a->ff_dim % 64) return HDIT_EUNSUPPORTED;
  if (!a->hidden || !a->encoder || !a->temb || !a->hidden_out || !a->encoder_out) return HDIT_EINVAL;
  if (!a->norm1_w || !a->norm1_b || !a->norm2_w || !a->norm2_b || !a->qkv_w || !a->to_out_w || !a->ff_in_w || !a->ff_out_w)
    return HDIT_EINVAL;
  if ((a->rope_cos == nullptr) != (a->rope_sin == nullptr)) return HDIT_EINVAL;
  if (a->fp8_attention != 0 && a->fp8_attention != 1) return HDIT_EINVAL;
  if (a->fp8_attention && cog_fp8_bytes(a) < 0) return HDIT_EINVAL;
  return HDIT_OK;
}

template <class Args>
int check_workspace(const Args* a, int64_t need) {
  if (!a->workspace || (((uintptr_t)a->workspace) & (ALIGN - 1)) || a->workspace_bytes < need) return HDIT_EINVAL;
  return HDIT_OK;
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int64_t hdit_block_flux_double_workspace_bytes(const hdit_flux_double_block_args* a) {
  return validate(a) == HDIT_OK ? carve(a, nullptr).bytes : -1;
}

extern "C" __attribute__((visibility("default"))) int hdit_block_flux_double(const hdit_flux_double_block_args* a, void* stream) {
  int rc = validate(a);
  if (rc != HDIT_OK) return rc;
  const FluxDoubleWs ws = carve(a, a->workspace);
  if ((rc = check_workspace(a, ws.bytes))) return rc;
  const hdit_sd3_block_weights& w = a->w;
  const int B = a->batch, Ni = a->n_img, Nt = a->n_txt, D = a->dim, F = a->ff_dim, H = a->heads, hd = D / H;
  const float eps = 1e-6f;
  const int64_t md = 6 * (int64_t)D;
  const float *ei = a->modulation_img, *et = a->modulation_txt;  // shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp
  if (!ei) {
    if ((rc = hdit_adaln_gemv(a->temb, w.norm1_w, w.norm1_b, ws.emb_img, B, 6 * D, a->temb_dim, stream))) return rc;
    ei = ws.emb_img;
  }
  if (!et) {
    if ((rc = hdit_adaln_gemv(a->temb, w.norm1_context_w, w.norm1_context_b, ws.emb_txt, B, 6 * D, a->temb_dim, stream))) return rc;
    et = ws.emb_txt;
  }
  hdit_ln_job jobs[2];
  ln_job(jobs[0], a->hidden, a->hidden_f32, ws.n_img, (int64_t)Ni * D, ei, ei + D, md, B, Ni, D);
  ln_job(jobs[1], a->encoder, a->encoder_f32, ws.n_txt, (int64_t)Nt * D, et, et + D, md, B, Nt, D);
  if ((rc = hdit_layernorm_modulate_jobs(jobs, 2, D, nullptr, nullptr, eps, stream))) return rc;
  hdit_gemm_problem probs[HDIT_GEMM_MAX_PROBLEMS];
  const int64_t ld3 = 3 * (int64_t)D, ld2 = 2 * (int64_t)D;
  // image q | k | v: one packed tensor, or (K/V buffer given) q alone and k | v straight into this call's rows of
  // the buffer, one problem per batch element (the destinations differ in batch stride)
  unsigned char *q_img = ws.qkv_img, *k_img, *v_img, *k_new;
  int64_t ld_q, ld_kv, kv_batch_rows;
  int kv_len, np = 0;
  if (a->kv_buffer) {
    unsigned char* buf = (unsigned char*)a->kv_buffer;
    const unsigned char* wkv = (const unsigned char*)w.qkv_w + (int64_t)D * D * 2;
    const unsigned char* bkv = w.qkv_b ? (const unsigned char*)w.qkv_b + (int64_t)D * 2 : nullptr;
    probs[np++] = problem(ws.n_img, D, w.qkv_w, w.qkv_b, q_img, D, B * Ni, D, D, HDIT_EPI_BIAS);
    for (int b = 0; b < B; b++)
      probs[np++] = problem(ws.n_img + (int64_t)b * Ni * D * 2, D, wkv, bkv,
                            buf + ((int64_t)b * a->kv_rows + a->kv_row0) * ld2 * 2, ld2, Ni, 2 * D, D, HDIT_EPI_BIAS);
    k_img = buf, v_img = buf + (int64_t)D * 2, k_new = buf + (int64_t)a->kv_row0 * ld2 * 2;
    ld_q = D, ld_kv = ld2, kv_batch_rows = a->kv_rows, kv_len = a->kv_rows;
  } else {
    probs[np++] = problem(ws.n_img, D, w.qkv_w, w.qkv_b, ws.qkv_img, 3 * D, B * Ni, 3 * D, D, HDIT_EPI_BIAS);
    k_img = ws.qkv_img + (int64_t)D * 2, v_img = ws.qkv_img + (int64_t)2 * D * 2, k_new = k_img;
    ld_q = ld3, ld_kv = ld3, kv_batch_rows = Ni, kv_len = Ni;
  }
  probs[np++] = problem(ws.n_txt, D, w.add_qkv_w, w.add_qkv_b, ws.qkv_txt, 3 * D, B * Nt, 3 * D, D, HDIT_EPI_BIAS);
  if ((rc = hdit_gemm_bf16(probs, np, stream))) return rc;
  // per-head RMSNorm on q, k of both streams, then the rotation of the joint [text, image] rows
  unsigned char *q_txt = ws.qkv_txt, *k_txt = ws.qkv_txt + (int64_t)D * 2, *v_txt = ws.qkv_txt + (int64_t)2 * D * 2;
  const float* cos_i = a->rope_cos ? a->rope_cos + (int64_t)Nt * hd : nullptr;
  const float* sin_i = a->rope_sin ? a->rope_sin + (int64_t)Nt * hd : nullptr;
  hdit_qknorm_job qj[4];
  qk_job(qj[0], q_txt, Nt, ld3, hd, a->norm_added_q_w, nullptr, a->rope_cos, a->rope_sin, Nt, 0, Nt, a->qk_norm_kind);
  qk_job(qj[1], k_txt, Nt, ld3, hd, a->norm_added_k_w, nullptr, a->rope_cos, a->rope_sin, Nt, 0, Nt, a->qk_norm_kind);
  qk_job(qj[2], q_img, Ni, ld_q, hd, a->norm_q_w, nullptr, cos_i, sin_i, Ni, 0, Ni, a->qk_norm_kind);
  qk_job(qj[3], k_new, kv_batch_rows, ld_kv, hd, a->norm_k_w, nullptr, cos_i, sin_i, Ni, 0, Ni, a->qk_norm_kind);
  if ((rc = hdit_qk_norm_rope(qj, 4, B, H, hd, a->qk_norm_eps, stream))) return rc;
  hdit_attn_args at;
  memset(&at, 0, sizeof(at));
  seg(at.q[0], q_txt, Nt, ld3, hd, Nt), seg(at.q[1], q_img, Ni, ld_q, hd, Ni);
  seg(at.k[0], k_txt, Nt, ld3, hd, Nt), seg(at.k[1], k_img, kv_batch_rows, ld_kv, hd, kv_len);
  seg(at.v[0], v_txt, Nt, ld3, hd, Nt), seg(at.v[1], v_img, kv_batch_rows, ld_kv, hd, kv_len);
  seg(at.o[0], ws.o_txt, Nt, D, hd, Nt), seg(at.o[1], ws.o_img, Ni, D, hd, Ni);
  at.batch = B, at.heads = H, at.head_dim = hd, at.scale = 0.f;
  if ((rc = hdit_attn_fwd_bf16(&at, stream))) return rc;
  // the reference's wrapper never adds the text out-projection bias back in its Flux branch
  // (layers/attention_processor.py:176-192,:284-305): to_add_out runs without bias
  probs[0] = problem(ws.o_img, D, w.to_out_w, w.to_out_b, ws.x1_img, D, B * Ni, D, D, 0);
  gated(probs[0], a->hidden, a->hidden_f32, ei + 2 * D, md, Ni, 1);
  probs[1] = problem(ws.o_txt, D, w.to_add_out_w, nullptr, ws.x1_txt, D, B * Nt, D, D, 0);
  gated(probs[1], a->encoder, a->encoder_f32, et + 2 * D, md, Nt, 1);
  if ((rc = hdit_gemm_bf16(probs, 2, stream))) return rc;
  ln_job(jobs[0], ws.x1_img, 1, ws.n_img, (int64_t)Ni * D, ei + 3 * D, ei + 4 * D, md, B, Ni, D);
  ln_job(jobs[1], ws.x1_txt, 1, ws.n_txt, (int64_t)Nt * D, et + 3 * D, et + 4 * D, md, B, Nt, D);
  if ((rc = hdit_layernorm_modulate_jobs(jobs, 2, D, nullptr, nullptr, eps, stream))) return rc;
  probs[0] = problem(ws.n_img, D, w.ff_in_w, w.ff_in_b, ws.h_img, F, B * Ni, F, D, HDIT_EPI_BIAS_GELU);
  probs[1] = problem(ws.n_txt, D, w.ff_context_in_w, w.ff_context_in_b, ws.h_txt, F, B * Nt, F, D, HDIT_EPI_BIAS_GELU);
  if ((rc = hdit_gemm_bf16(probs, 2, stream))) return rc;
  probs[0] = problem(ws.h_img, F, w.ff_out_w, w.ff_out_b, a->hidden_out, D, B * Ni, D, F, 0);
  gated(probs[0], ws.x1_img, 1, ei + 5 * D, md, Ni, a->out_f32);
  probs[1] = problem(ws.h_txt, F, w.ff_context_out_w, w.ff_context_out_b, a->encoder_out, D, B * Nt, D, F, 0);
  gated(probs[1], ws.x1_txt, 1, et + 5 * D, md, Nt, a->out_f32);
  return hdit_gemm_bf16(probs, 2, stream);
}

extern "C" __attribute__((visibility("default"))) int64_t hdit_block_flux_single_workspace_bytes(const hdit_flux_single_block_args* a) {
  return validate(a) == HDIT_OK ? carve(a, nullptr).bytes : -1;
}

extern "C" __attribute__((visibility("default"))) int hdit_block_flux_single(const hdit_flux_single_block_args* a, void* stream) {
  int rc = validate(a);
  if (rc != HDIT_OK) return rc;
  const FluxSingleWs ws = carve(a, a->workspace);
  if ((rc = check_workspace(a, ws.bytes))) return rc;
  const int B = a->batch, S = a->seq, D = a->dim, F = a->ff_dim, H = a->heads, hd = D / H;
  const int64_t md = 3 * (int64_t)D, ldc = (int64_t)D + F, ld3 = 3 * (int64_t)D;
  const float* emb = a->modulation;  // shift, scale, gate
  if (!emb) {
    if ((rc = hdit_adaln_gemv(a->temb, a->norm_w, a->norm_b, ws.emb, B, 3 * D, a->temb_dim, stream))) return rc;
    emb = ws.emb;
  }
  hdit_ln_job job;
  ln_job(job, a->hidden, a->hidden_f32, ws.n, (int64_t)S * D, emb, emb + D, md, B, S, D);
  if ((rc = hdit_layernorm_modulate_jobs(&job, 1, D, nullptr, nullptr, 1e-6f, stream))) return rc;
  // q|k|v and the MLP-in projection share their input: one launch; GELU(MLP) lands beside the attention output
  hdit_gemm_problem probs[HDIT_GEMM_MAX_PROBLEMS];
  hdit_qknorm_job qj[3];
  hdit_attn_args at;
  memset(&at, 0, sizeof(at));
  int np = 0, nj = 0;
  if (a->kv_buffer) {
    // patch mode: the queries of all rows in one [B, S, D] tensor, the text rows' k | v in a small tensor of their
    // own, the image rows' k | v straight into this patch's rows of the layer's buffer (one problem per batch element
    // and destination: the destinations differ in batch stride)
    const int Nt = a->n_txt, Ni = S - Nt;
    const int64_t ld2 = 2 * (int64_t)D;
    unsigned char* buf = (unsigned char*)a->kv_buffer;
    const unsigned char* wkv = (const unsigned char*)a->qkv_w + (int64_t)D * D * 2;
    const unsigned char* bkv = a->qkv_b ? (const unsigned char*)a->qkv_b + (int64_t)D * 2 : nullptr;
    probs[np++] = problem(ws.n, D, a->qkv_w, a->qkv_b, ws.qkv, D, B * S, D, D, HDIT_EPI_BIAS);
    for (int b = 0; b < B; b++) {
      const unsigned char* xb = ws.n + (int64_t)b * S * D * 2;
      if (Nt > 0)
        probs[np++] = problem(xb, D, wkv, bkv, ws.kv_txt + (int64_t)b * Nt * ld2 * 2, ld2, Nt, 2 * D, D, HDIT_EPI_BIAS);
      probs[np++] = problem(xb + (int64_t)Nt * D * 2, D, wkv, bkv, buf + ((int64_t)b * a->kv_rows + a->kv_row0) * ld2 * 2, ld2,
                            Ni, 2 * D, D, HDIT_EPI_BIAS);
    }
    const float* cos_i = a->rope_cos ? a->rope_cos + (int64_t)Nt * hd : nullptr;
    const float* sin_i = a->rope_sin ? a->rope_sin + (int64_t)Nt * hd : nullptr;
    qk_job(qj[nj++], ws.qkv, S, D, hd, a->norm_q_w, nullptr, a->rope_cos, a->rope_sin, S, 0, S, a->qk_norm_kind);
    if (Nt > 0)
      qk_job(qj[nj++], ws.kv_txt, Nt, ld2, hd, a->norm_k_w, nullptr, a->rope_cos, a->rope_sin, Nt, 0, Nt, a->qk_norm_kind);
    qk_job(qj[nj++], buf + (int64_t)a->kv_row0 * ld2 * 2, a->kv_rows, ld2, hd, a->norm_k_w, nullptr, cos_i, sin_i, Ni, 0, Ni,
           a->qk_norm_kind);
    seg(at.q[0], ws.qkv, S, D, hd, S);
    seg(at.k[0], ws.kv_txt, Nt, ld2, hd, Nt), seg(at.k[1], buf, a->kv_rows, ld2, hd, a->kv_rows);
    seg(at.v[0], ws.kv_txt + (int64_t)D * 2, Nt, ld2, hd, Nt), seg(at.v[1], buf + (int64_t)D * 2, a->kv_rows, ld2, hd, a->kv_rows);
  } else {
    unsigned char *q = ws.qkv, *k = ws.qkv + (int64_t)D * 2, *v = ws.qkv + (int64_t)2 * D * 2;
    probs[np++] = problem(ws.n, D, a->qkv_w, a->qkv_b, ws.qkv, ld3, B * S, 3 * D, D, HDIT_EPI_BIAS);
    qk_job(qj[nj++], q, S, ld3, hd, a->norm_q_w, nullptr, a->rope_cos, a->rope_sin, S, 0, S, a->qk_norm_kind);
    qk_job(qj[nj++], k, S, ld3, hd, a->norm_k_w, nullptr, a->rope_cos, a->rope_sin, S, 0, S, a->qk_norm_kind);
    seg(at.q[0], q, S, ld3, hd, S), seg(at.k[0], k, S, ld3, hd, S), seg(at.v[0], v, S, ld3, hd, S);
  }
  probs[np++] = problem(ws.n, D, a->proj_mlp_w, a->proj_mlp_b, ws.cat + (int64_t)D * 2, ldc, B * S, F, D, HDIT_EPI_BIAS_GELU);
  if ((rc = hdit_gemm_bf16(probs, np, stream))) return rc;
  if ((rc = hdit_qk_norm_rope(qj, nj, B, H, hd, a->qk_norm_eps, stream))) return rc;
  seg(at.o[0], ws.cat, S, ldc, hd, S);
  at.batch = B, at.heads = H, at.head_dim = hd, at.scale = 0.f;
  if ((rc = hdit_attn_fwd_bf16(&at, stream))) return rc;
  probs[0] = problem(ws.cat, ldc, a->proj_out_w, a->proj_out_b, a->hidden_out, D, B * S, D, D + F, 0);
  gated(probs[0], a->hidden, a->hidden_f32, emb + 2 * D, md, S, a->out_f32);
  return hdit_gemm_bf16(probs, 1, stream);
}

extern "C" __attribute__((visibility("default"))) int64_t hdit_block_cogvideox_workspace_bytes(const hdit_cogvideox_block_args* a) {
  return validate(a) == HDIT_OK ? carve(a, nullptr).bytes : -1;
}

extern "C" __attribute__((visibility("default"))) int hdit_block_cogvideox(const hdit_cogvideox_block_args* a, void* stream) {
  int rc = validate(a);
  if (rc != HDIT_OK) return rc;
  const CogWs ws = carve(a, a->workspace);
  if ((rc = check_workspace(a, ws.bytes))) return rc;
  const int B = a->batch, N = a->n_img, Nt = a->n_txt, S = N + Nt, D = a->dim, F = a->ff_dim, H = a->heads, hd = D / H;
  const int64_t md = 6 * (int64_t)D, ld3 = 3 * (int64_t)D;
  const int sz_h = a->hidden_f32 ? 4 : 2, sz_e = a->encoder_f32 ? 4 : 2, sz_o = a->out_f32 ? 4 : 2;
  // norm1: chunks shift, scale, gate, enc_shift, enc_scale, enc_gate; one affine LayerNorm for both streams,
  // both results written into one joint [text, video] buffer
  const float *e1 = a->modulation1, *e2 = a->modulation2;
  if (!e1) {
    if ((rc = hdit_adaln_gemv(a->temb, a->norm1_w, a->norm1_b, ws.emb1, B, 6 * D, a->temb_dim, stream))) return rc;
    e1 = ws.emb1;
  }
  if (!e2) {
    if ((rc = hdit_adaln_gemv(a->temb, a->norm2_w, a->norm2_b, ws.emb2, B, 6 * D, a->temb_dim, stream))) return rc;
    e2 = ws.emb2;
  }
  hdit_ln_job jobs[2];
  ln_job(jobs[0], a->encoder, a->encoder_f32, ws.joint, (int64_t)S * D, e1 + 3 * D, e1 + 4 * D, md, B, Nt, D);
  ln_job(jobs[1], a->hidden, a->hidden_f32, ws.joint + (int64_t)Nt * D * 2, (int64_t)S * D, e1, e1 + D, md, B, N, D);
  if ((rc = hdit_layernorm_modulate_jobs(jobs, 2, D, a->norm1_ln_w, a->norm1_ln_b, a->norm_eps, stream))) return rc;
  hdit_gemm_problem probs[HDIT_GEMM_MAX_PROBLEMS];
  probs[0] = problem(ws.joint, D, a->qkv_w, a->qkv_b, ws.qkv, ld3, B * S, 3 * D, D, HDIT_EPI_BIAS);
  if ((rc = hdit_gemm_bf16(probs, 1, stream))) return rc;
  unsigned char *q = ws.qkv, *k = ws.qkv + (int64_t)D * 2, *v = ws.qkv + (int64_t)2 * D * 2;
  if (a->qk_norm_kind || a->rope_cos) {
    hdit_qknorm_job qj[2];
    qk_job(qj[0], q, S, ld3, hd, a->norm_q_w, a->norm_q_b, a->rope_cos, a->rope_sin, S, Nt, N, a->qk_norm_kind);
    qk_job(qj[1], k, S, ld3, hd, a->norm_k_w, a->norm_k_b, a->rope_cos, a->rope_sin, S, Nt, N, a->qk_norm_kind);
    if ((rc = hdit_qk_norm_rope(qj, 2, B, H, hd, a->qk_norm_eps, stream))) return rc;
  }
  hdit_attn_args at;
  cog_attn_args(a, at, q, k, v, ws.o);
  if (a->fp8_attention) {
    if ((rc = hdit_attn_absmax(&at, ws.absmax, stream))) return rc;
    if ((rc = hdit_attn_fwd_fp8(&at, ws.absmax, ws.fp8, stream))) return rc;
  } else if ((rc = hdit_attn_fwd_bf16(&at, stream))) {
    return rc;
  }
  // one weight set over the joint rows, per-stream gates: per batch element a text and a video problem
  auto gated_pair = [&](const unsigned char* a_joint, int64_t lda, const void* wt, const void* bias, int kdim, const void* res_e,
                        int re_sz, const void* res_h, int rh_sz, const float* emb, void* out_e, int oe_sz, void* out_h, int oh_sz) {
    int np = 0;
    for (int b = 0; b < B; b++) {
      const unsigned char* ab = a_joint + (int64_t)b * S * lda * 2;
      probs[np] = problem(ab, lda, wt, bias, (unsigned char*)out_e + (int64_t)b * Nt * D * oe_sz, D, Nt, D, kdim, 0);
      gated(probs[np++], (const unsigned char*)res_e + (int64_t)b * Nt * D * re_sz, re_sz == 4, emb + b * md + 5 * D, md, Nt, oe_sz == 4);
      probs[np] = problem(ab + (int64_t)Nt * lda * 2, lda, wt, bias, (unsigned char*)out_h + (int64_t)b * N * D * oh_sz, D, N, D, kdim, 0);
      gated(probs[np++], (const unsigned char*)res_h + (int64_t)b * N * D * rh_sz, rh_sz == 4, emb + b * md + 2 * D, md, N, oh_sz == 4);
    }
    return hdit_gemm_bf16(probs, np, stream);
  };
  if ((rc = gated_pair(ws.o, D, a->to_out_w, a->to_out_b, D, a->encoder, sz_e, a->hidden, sz_h, e1, ws.x1_e, 4, ws.x1_h, 4))) return rc;
  ln_job(jobs[0], ws.x1_e, 1, ws.joint, (int64_t)S * D, e2 + 3 * D, e2 + 4 * D, md, B, Nt, D);
  ln_job(jobs[1], ws.x1_h, 1, ws.joint + (int64_t)Nt * D * 2, (int64_t)S * D, e2, e2 + D, md, B, N, D);
  if ((rc = hdit_layernorm_modulate_jobs(jobs, 2, D, a->norm2_ln_w, a->norm2_ln_b, a->norm_eps, stream))) return rc;
  probs[0] = problem(ws.joint, D, a->ff_in_w, a->ff_in_b, ws.h, F, B * S, F, D, HDIT_EPI_BIAS_GELU);
  if ((rc = hdit_gemm_bf16(probs, 1, stream))) return rc;
  return gated_pair(ws.h, F, a->ff_out_w, a->ff_out_b, F, ws.x1_e, 4, ws.x1_h, 4, e2, a->encoder_out, sz_o, a->hidden_out, sz_o);
}
