#include "stack_executor.h"

#include <stdexcept>
#include <string>

namespace omx {
namespace stack {

static void need(bool ok, const std::string& what) {
  if (!ok) throw std::runtime_error("stack executor: " + what);
}

void StackExecutor::validate() const {
  need(cfg.E > 0 && cfg.V > 0 && cfg.max_B > 0, "not configured");
  need(embed_w && final_w && final_b && head_w, "global weights missing");
  need(ws.resid && ws.x0 && ws.h && ws.proj && ws.a && ws.y && ws.lrows, "workspace missing");
  need(in.tokens && in.pos && in.slot && in.q_len && in.q_seq && in.block_table && in.logits, "step inputs missing");
  need(!runs.empty(), "no layer runs");
  for (const RunDesc& r : runs) {
    need(r.layer >= 0 && r.layer < (int)layers.size(), "a run names a layer that does not exist");
    const LayerDesc& L = layers[r.layer];
    need(L.norm_w && L.norm_b && L.w_in && L.w_o && L.n_in > 0 && L.n_in <= ws.ld_proj, "layer weights missing");
    need(L.heads * L.vdim <= ws.ld_a, "mixer output wider than its buffer");
    if (r.opens_pass) need(loop_in && ws.cat, "the pass-opening projection is missing");
    if (L.kind == 0) {
      need(r.kc && r.vc, "attention run without a K/V pool");
      need(L.dim <= 256 && L.vdim <= 256 && L.kv_heads > 0 && L.heads % L.kv_heads == 0, "attention head sizes");
    } else {
      need(r.state && L.decay, "retention run without a state");
      need(retention_supported(L.dim, L.vdim) || retention_general_supported(L.dim, L.vdim), "retention head sizes (<= 1024)");
      need(L.rot_dims == 0 || L.inv_freq, "retention rotary table missing");
    }
    if (L.experts) {
      need(L.top > 0 && L.top <= MOE_MAX_TOP && L.top <= ws.ld_top && L.top * L.ff + L.shared_ff <= ws.ld_hmid && ws.hmid &&
               ws.eids && ws.ew && L.router_b && L.w_gu && L.w_down && (!L.shared_ff || (L.sh_down && ws.sgate)),
           "routed feed-forward sizes");
    }
  }
}

void StackExecutor::embed(int B, hipStream_t s) {
  stack::embed(embed_w, in.tokens, B, cfg.E, cfg.V, ws.resid, ws.x0, cfg.f32, s);
}

void StackExecutor::layer_run(int ri, int B, hipStream_t s) {
  const RunDesc& r = runs.at(ri);
  const LayerDesc& L = layers[r.layer];
  const int E = cfg.E, f32 = cfg.f32;
  if (r.opens_pass) {
    concat_cast(ws.resid, ws.x0, B, E, ws.cat, f32, s);
    GemmParams g{ws.cat, 2 * E, loop_in, B, E, 2 * E, ws.resid, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  StepRows R{B, in.pos, in.slot, in.q_len, in.q_seq, in.block_table, in.max_blocks, in.bs};
  AttnParams A{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.heads, L.kv_heads, L.dim, L.vdim, L.scale, L.softcap,
               L.qtemp_coef, L.qtemp_every, r.kc, r.vc, ws.a, ws.ld_a, f32, n_splits, ws.split_ws, ws.split_ws_floats};
  const bool fused_in = gemv_ln_supported(B, E, f32);
  if (fused_in) {  // decode steps: norm + input projection (+ query temperature and K/V store) in one launch
    gemv_ln(ws.resid, E, L.norm_w, L.norm_b, cfg.eps, L.w_in, B, L.n_in, ws.proj, ws.ld_proj, ws.h, L.kind == 0 ? &A : nullptr,
            &R, f32, s);
  } else {
    layer_norm_cast(ws.resid, nullptr, B, E, L.norm_w, L.norm_b, cfg.eps, ws.h, f32, s);
    // every matrix that reads the normed activations, in one product
    GemmParams g{ws.h, E, L.w_in, B, L.n_in, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  if (L.kind == 0) {
    if (!fused_in) attn_prepare(A, R, s);
    if (B > SMALL_B && n_tiles > 0 && tiles && flash_prefill_supported(A))
      flash_prefill(A, R, tiles, n_tiles, s);  // prompt portions: query tiles on the matrix cores
    else
      attention(A, R, s);
  } else {
    RetParams P{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.off_g, L.heads, L.dim, L.vdim, L.rot_dims, L.inv_freq,
                L.decay, r.state, cfg.eps, ws.a, ws.ld_a, f32};
    // prompt portions in chunks (the host bound this step's chunk table); else token by token in one launch
    if (B > SMALL_B && n_chunks > 0 && ws.ret.U && ws.ret.ld_o >= L.heads * L.vdim &&
        ws.ret.u_stride >= (long long)L.heads * L.dim * L.vdim && retention_chunk_supported(L.dim, L.vdim)) {
      RetChunkWs W = ws.ret;
      W.nchunks = n_chunks;
      retention_chunked(P, R, W, s);
    } else
      retention(P, R, s);
  }
  const float* ff = nullptr;
  if (L.experts) {
    MoeParams M{ws.proj, ws.ld_proj, L.off_router, L.off_sg, L.off_sgate, L.off_sup, B, E, L.experts, L.top, L.ff,
                L.shared_ff, L.router_b, ws.h, L.w_gu, L.w_down, L.sh_down, ws.eids, ws.ew, ws.ld_top, ws.sgate, ws.hmid,
                ws.ld_hmid, ws.y, f32};
    if (B <= SMALL_B) {  // decode steps: two launches end the layer (residual update included)
      moe_fused_small(M, ws.a, ws.ld_a, L.w_o, L.heads * L.vdim, ws.resid, cfg.residual_mult, s);
      return;
    }
    moe_route(M, s);
    if (ws.moe.gu && moe_grouped_supported(M)) {
      moe_grouped(M, ws.moe, s);  // rows sorted by expert, one matrix-core product per expert tile
    } else {
      moe_experts(M, s);          // every pair streams its expert's rows once
      moe_down(M, s);
    }
    ff = ws.y;
  }
  // x <- x + m * (mixer output projection + feed-forward)
  GemmParams o{ws.a, ws.ld_a, L.w_o, B, E, L.heads * L.vdim, ws.resid, E, EPI_RESID, cfg.residual_mult, ff, 0.f, f32};
  gemm(o, s);
}

void StackExecutor::head(int n_logits, bool use_idx, hipStream_t s) {
  if (n_logits <= 0) return;
  layer_norm_cast(ws.resid, use_idx ? in.logit_idx : nullptr, n_logits, cfg.E, final_w, final_b, cfg.eps, ws.lrows, cfg.f32,
                  s);
  GemmParams g{ws.lrows, cfg.E, head_w, n_logits, cfg.V, cfg.E, in.logits, in.ld_logits, EPI_SOFTCAP, 0.f, nullptr,
               cfg.logit_softcap, cfg.f32};
  gemm(g, s);
}

void StackExecutor::forward(int B, int n_logits, bool use_idx, hipStream_t s) {
  embed(B, s);
  for (int ri = 0; ri < (int)runs.size(); ++ri) layer_run(ri, B, s);
  head(n_logits, use_idx, s);
}

}  // namespace stack
}  // namespace omx
