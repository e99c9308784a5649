// Whole-step executor of the Gezozen decoder family: layers listed in the model's configuration that normalise AFTER the sum and
// whose sublayers read the stream itself,
//   x <- N1(alpha x + sigmoid(R1 x + r1) * mixer(x));   x <- N2(alpha x + sigmoid(R2 x + r2) * ff(x));   logits = head . N(x)
// with N a root-mean-square norm over equal consecutive groups of the row (packed_ops.hip) and one alpha for the model.
// Mixers (every size and constant per layer):
//   VMX_MIXER_ATTENTION_GLA        left_scale * (grouped-query attention: per-head q / k norms, rotation in halves, soft-capped
//                                  scores, causal) + right_scale * (gated linear attention: S <- diag(a_t) S + k_t v_t^T with
//                                  a_t = sigmoid(W2 W1 x + b)^(1 / tau) per key channel, o_t = S^T q_t / sqrt(dim))
//   VMX_MIXER_ATTENTION_RETENTION  left_scale * (the same attention with biased projections, stretched rotation frequencies and a
//                                  sliding window) + right_scale * (retention: rotated q and k, one constant decay per head)
//   VMX_MIXER_HEAD_DELTA           short causal convolutions + SiLU on q, k, v, unit-vector q and k, gated delta rule with one decay
//                                  per head, exp(-exp(A) softplus(W_a x + dt))
// Every recurrent read-out is RMS-normed per head, multiplied by silu(W_g x) and projected.  The attention is window_attn.hip over
// a paged key/value cache, the three recurrences are ONE kernel (delta_rule.hip) over a matrix memory per head in the sequence's
// state slot, which also holds the convolutions' last inputs.
// Feed-forward VMX_MLP_SIGMOID_MOE: router scores sigmoid(W_r x), the `top` largest win and are NOT renormalised; the score
// multiplies the expert's INPUT (gate and up products are linear, so it is applied to their results: silu(s g) * (s u)); a shared
// expert runs for every token, times sigmoid(w_sg . x).  Experts run as token-grouped products over pairs sorted by expert.
//
// Every product that reads the mixer's input (q, k, v of both sides, output-gate and decay projections, the residual gate) is ONE
// linear whose f32 output row the other kernels address by column offset; the same for the feed-forward's input (shared gate | up,
// the shared expert's gate, the residual gate).  `acc` carries alpha * x and collects the gated sublayer results through the
// accumulating epilogue of the output projections; the norm kernel turns it into the next x, its copy for the linears (bf16 in
// VMX_BF16 mode) and the next alpha * x.  The stream, norms, router, positions and angles, scores, softmax, decays, gates of the
// recurrences and their state are f32 in both modes; VMX_BF16 rounds the operands of the linears and the cache rows to bf16,
// VMX_F32 multiplies in true f32 everywhere.  The forward call allocates nothing, reads nothing back and is graph-capturable.
#include "vmx_kernels.h"
#include <math.h>
#include <algorithm>
#include <string>
#include <vector>

namespace {

using Buf = VmxBuf;

int pad8(int n) { return (n + 7) & ~7; }

struct Seg {       // where a checkpoint tensor lands: rows of a fused projection, or a buffer of its own
    Buf *buf = nullptr;
    size_t offset = 0, bytes = 0;
};

struct Layer {
    vmx_gezozen_layer_config c;
    Buf norm1, norm2, wfused, bias, wfused2, bias2;
    Buf qnorm, knorm, wo, rot_steps, kcache, vcache;                                // attention
    Buf wo_right, onorm, wa2, a2b, decay, r_rot_steps, s_state;                     // recurrent side
    Buf conv_taps, a_log, dt_bias, conv_state;                                      // delta
    Buf router, egu, edown, sdown;                                                  // feed-forward
    float rot_mul = 1.f, r_rot_mul = 1.f;
    int nf = 0, q_off = 0, k_off = 0, v_off = 0, rq_off = 0, rk_off = 0, rv_off = 0, g_off = 0, a1_off = 0, b_off = 0, a_off = 0, rg1_off = 0;
    int nf2 = 0, sgu_off = 0, sg_off = 0, rg2_off = 0;
    int rh = 0, rqk = 0, rd = 0, rv = 0;   // the recurrence as it runs: value heads, query/key heads, key size, value size
    std::vector<std::pair<std::string, Seg>> tensors;   // checkpoint name (without the layer prefix) -> destination
    std::vector<std::string> missing;
    void want(const std::string &name, Buf *b, size_t off, size_t bytes) {
        tensors.push_back({name, Seg{b, off, bytes}});
        missing.push_back(name);
    }
};

}  // namespace

struct vmx_gezozen {
    vmx_gezozen_config cfg;
    std::vector<Layer> layers;
    Buf embed, final_norm, head;
    std::vector<std::string> missing;
    Buf x, acc, h, hsel, fused, qbuf, attn, attn_ws, conv, dec, dro, rec, argmax_keys;
    Buf few_pairs, rlogits, topw, topi, sorted, blk_expert, total, inv, gu, act, ydown, sact, sout;
    bool f32() const { return cfg.dtype == VMX_F32; }
    size_t esz() const { return f32() ? 4 : 2; }
};

namespace {

int upload(Buf &b, size_t offset, const void *data, size_t bytes, hipStream_t st) {
    VMX_CHECK_HIP(hipMemcpyAsync((char *)b.p + offset, data, bytes, hipMemcpyDefault, st));
    VMX_CHECK_HIP(hipStreamSynchronize(st));
    return VMX_OK;
}

void erase_name(std::vector<std::string> &v, const std::string &n) {
    for (size_t i = 0; i < v.size(); i++)
        if (v[i] == n) {
            v.erase(v.begin() + i);
            return;
        }
}

int alloc_zero(Buf &b, size_t n) {
    if (int rc = b.alloc(n)) return rc;
    VMX_CHECK_HIP(hipMemset(b.p, 0, n ? n : 16));
    return VMX_OK;
}

bool rotation_ok(const vmx_rotation &r, int head_dim) {
    if (r.dims == 0) return true;
    if (r.dims < 0 || r.dims % 2 || r.dims > head_dim || !(r.base > 1.0)) return false;
    return r.factor == 0.0 || (r.factor > 0.0 && r.original > 0.0 && r.fast > 0.0 && r.slow > 0.0);
}

int upload_rotation(const vmx_rotation &r, Buf &steps, float &mul) {
    mul = 1.f;
    if (r.dims <= 0) return VMX_OK;
    std::vector<float> f(r.dims / 2);
    if (int rc = vmx_rotation_steps(&r, f.data(), &mul)) return rc;
    if (int rc = steps.alloc(f.size() * 4)) return rc;
    VMX_CHECK_HIP(hipMemcpy(steps.p, f.data(), f.size() * 4, hipMemcpyHostToDevice));
    return VMX_OK;
}

}  // namespace

extern "C" int vmx_rotation_steps(const vmx_rotation *rot, float *steps, float *mul) {
    VMX_REQUIRE(rot && steps && mul, "rotation_steps: null pointer");
    const vmx_rotation &r = *rot;
    VMX_REQUIRE(r.dims >= 2 && r.dims % 2 == 0 && r.base > 1.0, "rotation_steps: %d rotated coordinates, base %g", r.dims, r.base);
    const int half = r.dims / 2;
    *mul = 1.f;
    double lo = 0, hi = 0;
    if (r.factor > 0.0) {
        VMX_REQUIRE(r.original > 0.0 && r.fast > 0.0 && r.slow > 0.0, "rotation_steps: bad stretch constants");
        auto idx = [&](double turns) { return r.dims * log(r.original / (2.0 * M_PI * turns)) / (2.0 * log(r.base)); };
        lo = std::max(floor(idx(r.fast)), 0.0);
        hi = std::min(ceil(idx(r.slow)), (double)(r.dims - 1));
        *mul = (float)(0.1 * log(r.factor) + 1.0);
    }
    for (int i = 0; i < half; i++) {
        double f = pow(r.base, -2.0 * i / r.dims);
        if (r.factor > 0.0) {
            const double ramp = std::min(std::max((i - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
            f = f / r.factor * ramp + f * (1.0 - ramp);
        }
        steps[i] = (float)f;
    }
    return VMX_OK;
}

extern "C" int vmx_gezozen_create(const vmx_gezozen_config *cfg, const vmx_gezozen_layer_config *layer_cfgs, vmx_gezozen **out) {
    VMX_REQUIRE(cfg && layer_cfgs && out, "gezozen_create: null pointer");
    const vmx_gezozen_config &c = *cfg;
    VMX_REQUIRE(c.vocab >= 1 && c.width >= 1 && c.num_layers >= 1, "gezozen_create: bad sizes (vocab %d, width %d, layers %d)", c.vocab, c.width,
                c.num_layers);
    VMX_REQUIRE(c.norm_groups >= 1 && c.width % c.norm_groups == 0, "gezozen_create: %d norm groups do not divide the width %d", c.norm_groups,
                c.width);
    VMX_REQUIRE(c.dtype == VMX_F32 || c.dtype == VMX_BF16, "gezozen_create: dtype must be VMX_F32 or VMX_BF16");
    VMX_REQUIRE(c.block_size >= 1 && c.num_blocks >= 1 && c.max_tokens >= 1 && c.max_seqs >= 1 && c.state_slots >= 1,
                "gezozen_create: bad cache / batch geometry");
    vmx_gezozen *m = new vmx_gezozen();
    m->cfg = c;
    m->layers.resize(c.num_layers);
    const size_t T = c.max_tokens, W = c.width, rows = (size_t)c.num_blocks * c.block_size;
    size_t attn_ws = 16, nf = 8, hd = 1, hv = 1, convc = 1, rhd = 1, rhv = 1, ne = 1, pairs = 0, cap = (size_t)VMX_MOE_FEW_PAIRS * 16, eff = 1, sff = 1;
    int rc = VMX_OK;
#define GA(buf, n)                        \
    do {                                  \
        if (!rc) rc = alloc_zero(buf, n); \
    } while (0)
#define BAD(...)                    \
    {                               \
        vmx_set_error(__VA_ARGS__); \
        rc = VMX_EINVAL;            \
        break;                      \
    }
    for (int li = 0; li < c.num_layers && !rc; li++) {
        Layer &L = m->layers[li];
        L.c = layer_cfgs[li];
        L.c.decay = nullptr;   // host arrays of the caller are read here and not kept
        const vmx_gezozen_layer_config &lc = layer_cfgs[li];
        if (lc.heads < 1 || lc.kv_heads < 1 || lc.heads % lc.kv_heads || lc.dim < 1 || lc.dim > 256 || lc.vdim < 1 || lc.vdim > 256)
            BAD("gezozen_create: layer %d: bad head counts or sizes (heads %d, kv_heads %d, dim %d, vdim %d; sizes up to 256)", li, lc.heads,
                lc.kv_heads, lc.dim, lc.vdim);
        const bool ff = lc.mlp != VMX_MLP_NONE;
        const size_t H = lc.heads, G = lc.kv_heads, D = lc.dim, V = lc.vdim;
        int at = 0;
        auto seg = [&](int n) {
            const int o = at;
            at = pad8(at + n);
            return o;
        };
        L.want("norm1", &L.norm1, 0, W * 2);
        GA(L.norm1, W * 2);
        const bool two_sided = lc.mixer == VMX_MIXER_ATTENTION_GLA || lc.mixer == VMX_MIXER_ATTENTION_RETENTION;
        if (two_sided) {
            const bool gla = lc.mixer == VMX_MIXER_ATTENTION_GLA;
            if (lc.window < 0 || lc.softcap < 0.f) BAD("gezozen_create: layer %d: bad attention mask or soft cap", li);
            if (!rotation_ok(lc.rot, lc.dim)) BAD("gezozen_create: layer %d: bad rotation of the attention (%d coordinates in heads of %d)", li, lc.rot.dims, lc.dim);
            if (lc.r_heads < 1 || lc.r_dim < 1 || lc.r_dim > 256 || lc.r_vdim < 1)
                BAD("gezozen_create: layer %d: bad sizes of the recurrent side (heads %d, dim %d, vdim %d)", li, lc.r_heads, lc.r_dim, lc.r_vdim);
            if (gla && (!(lc.tau > 0.f) || lc.decay_rank < 1)) BAD("gezozen_create: layer %d: bad decay constants (tau %g, rank %d)", li, lc.tau, lc.decay_rank);
            if (!gla && (!lc.decay || !rotation_ok(lc.r_rot, lc.r_dim))) BAD("gezozen_create: layer %d: retention needs its decays and a valid rotation", li);
            const size_t RH = lc.r_heads, RD = lc.r_dim, RV = lc.r_vdim;
            L.rh = L.rqk = lc.r_heads, L.rd = lc.r_dim, L.rv = lc.r_vdim;
            L.q_off = seg(H * D);
            L.k_off = seg(G * D);
            L.v_off = seg(G * V);
            L.rq_off = seg(2 * RH * RD);   // q | k adjacent: one preparation launch rotates both
            L.rk_off = L.rq_off + RH * RD;
            L.rv_off = seg(RH * RV);
            L.g_off = seg(RH * RV);
            if (gla) L.a1_off = seg(lc.decay_rank);
            L.rg1_off = seg(W);
            L.nf = at;
            GA(L.wfused, (size_t)L.nf * W * 2);
            GA(L.bias, (size_t)L.nf * 2);
            GA(L.qnorm, D * 2);
            GA(L.knorm, D * 2);
            GA(L.wo, W * H * V * 2);
            GA(L.wo_right, W * RH * RV * 2);
            GA(L.kcache, rows * G * D * m->esz());
            GA(L.vcache, rows * G * V * m->esz());
            GA(L.s_state, vmx_gated_delta_rule_state_bytes(c.state_slots, lc.r_heads, lc.r_dim, lc.r_vdim));
            L.want("mix.left.q", &L.wfused, (size_t)L.q_off * W * 2, H * D * W * 2);
            L.want("mix.left.k", &L.wfused, (size_t)L.k_off * W * 2, G * D * W * 2);
            L.want("mix.left.v", &L.wfused, (size_t)L.v_off * W * 2, G * V * W * 2);
            if (lc.qkv_bias) {
                L.want("mix.left.q.b", &L.bias, (size_t)L.q_off * 2, H * D * 2);
                L.want("mix.left.k.b", &L.bias, (size_t)L.k_off * 2, G * D * 2);
                L.want("mix.left.v.b", &L.bias, (size_t)L.v_off * 2, G * V * 2);
            }
            L.want("mix.left.q.norm", &L.qnorm, 0, D * 2);
            L.want("mix.left.k.norm", &L.knorm, 0, D * 2);
            L.want("mix.left.o", &L.wo, 0, W * H * V * 2);
            L.want("mix.right.q", &L.wfused, (size_t)L.rq_off * W * 2, RH * RD * W * 2);
            L.want("mix.right.k", &L.wfused, (size_t)L.rk_off * W * 2, RH * RD * W * 2);
            L.want("mix.right.v", &L.wfused, (size_t)L.rv_off * W * 2, RH * RV * W * 2);
            L.want("mix.right.g", &L.wfused, (size_t)L.g_off * W * 2, RH * RV * W * 2);
            L.want("mix.right.o", &L.wo_right, 0, W * RH * RV * 2);
            if (gla) {
                GA(L.onorm, RV * 2);
                GA(L.wa2, RH * RD * lc.decay_rank * 2);
                GA(L.a2b, RH * RD * 2);
                L.want("mix.right.norm", &L.onorm, 0, RV * 2);
                L.want("mix.right.a1", &L.wfused, (size_t)L.a1_off * W * 2, (size_t)lc.decay_rank * W * 2);
                L.want("mix.right.a2", &L.wa2, 0, RH * RD * lc.decay_rank * 2);
                L.want("mix.right.a2.b", &L.a2b, 0, RH * RD * 2);
            } else {
                GA(L.decay, RH * 4);
                if (!rc && hipMemcpy(L.decay.p, lc.decay, RH * 4, hipMemcpyHostToDevice) != hipSuccess) BAD("gezozen_create: upload failed");
                if (!rc) rc = upload_rotation(lc.r_rot, L.r_rot_steps, L.r_rot_mul);
            }
            if (!rc) rc = upload_rotation(lc.rot, L.rot_steps, L.rot_mul);
            attn_ws = std::max(attn_ws, vmx_window_attention_workspace_bytes((int)T, lc.heads, lc.vdim));
            hd = std::max(hd, H * D);
            hv = std::max(hv, H * V);
            convc = std::max(convc, 2 * RH * RD);
        } else if (lc.mixer == VMX_MIXER_HEAD_DELTA) {
            if (lc.conv_taps < 1 || lc.conv_taps > 64) BAD("gezozen_create: layer %d: bad convolution length %d", li, lc.conv_taps);
            const size_t C = 2 * G * D + H * V, n = lc.conv_taps;
            L.rh = lc.heads, L.rqk = lc.kv_heads, L.rd = lc.dim, L.rv = lc.vdim;
            L.q_off = seg(2 * G * D + H * V);   // q | k | v stay adjacent: the convolution sees one run of channels
            L.k_off = L.q_off + G * D;
            L.v_off = L.k_off + G * D;
            L.b_off = seg(H);
            L.a_off = seg(H);
            L.g_off = seg(H * V);
            L.rg1_off = seg(W);
            L.nf = at;
            GA(L.wfused, (size_t)L.nf * W * 2);
            GA(L.bias, (size_t)L.nf * 2);
            GA(L.conv_taps, C * n * 2);
            GA(L.a_log, H * 2);
            GA(L.dt_bias, H * 2);
            GA(L.onorm, V * 2);
            GA(L.wo_right, W * H * V * 2);
            GA(L.conv_state, vmx_short_conv_state_bytes(c.state_slots, (int)C, lc.conv_taps));
            GA(L.s_state, vmx_gated_delta_rule_state_bytes(c.state_slots, lc.heads, lc.dim, lc.vdim));
            L.want("mix.q", &L.wfused, (size_t)L.q_off * W * 2, G * D * W * 2);
            L.want("mix.k", &L.wfused, (size_t)L.k_off * W * 2, G * D * W * 2);
            L.want("mix.v", &L.wfused, (size_t)L.v_off * W * 2, H * V * W * 2);
            L.want("mix.q.conv", &L.conv_taps, 0, G * D * n * 2);
            L.want("mix.k.conv", &L.conv_taps, G * D * n * 2, G * D * n * 2);
            L.want("mix.v.conv", &L.conv_taps, 2 * G * D * n * 2, H * V * n * 2);
            L.want("mix.b", &L.wfused, (size_t)L.b_off * W * 2, H * W * 2);
            L.want("mix.a", &L.wfused, (size_t)L.a_off * W * 2, H * W * 2);
            L.want("mix.A_log", &L.a_log, 0, H * 2);
            L.want("mix.dt_bias", &L.dt_bias, 0, H * 2);
            L.want("mix.norm", &L.onorm, 0, V * 2);
            L.want("mix.g", &L.wfused, (size_t)L.g_off * W * 2, H * V * W * 2);
            L.want("mix.o", &L.wo_right, 0, W * H * V * 2);
            convc = std::max(convc, C);
        } else {
            vmx_set_error("gezozen_create: layer %d: unknown mixer kind %d", li, lc.mixer);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        rhd = std::max(rhd, (size_t)L.rh * L.rd);
        rhv = std::max(rhv, (size_t)L.rh * L.rv);
        L.want("rg1", &L.wfused, (size_t)L.rg1_off * W * 2, W * W * 2);
        L.want("rg1.b", &L.bias, (size_t)L.rg1_off * 2, W * 2);
        if (lc.mlp == VMX_MLP_SIGMOID_MOE) {
            if (lc.experts < 1 || lc.experts > 256 || lc.top < 1 || lc.top > lc.experts || lc.expert_ff < 1 || lc.shared_ff < 0)
                BAD("gezozen_create: layer %d: bad mixture-of-experts sizes (1 .. 256 experts, top <= experts)", li);
            const size_t one = (size_t)lc.expert_ff * W * 2, S = lc.shared_ff;
            at = 0;
            if (S) {
                L.sgu_off = seg(2 * S);   // shared gate rows, then shared up rows
                L.sg_off = seg(1);
            }
            L.rg2_off = seg(W);
            L.nf2 = at;
            GA(L.norm2, W * 2);
            GA(L.wfused2, (size_t)L.nf2 * W * 2);
            GA(L.bias2, (size_t)L.nf2 * 2);
            GA(L.router, (size_t)lc.experts * W * 2);
            GA(L.egu, (size_t)lc.experts * 2 * one);
            GA(L.edown, (size_t)lc.experts * one);
            L.want("norm2", &L.norm2, 0, W * 2);
            L.want("rg2", &L.wfused2, (size_t)L.rg2_off * W * 2, W * W * 2);
            L.want("rg2.b", &L.bias2, (size_t)L.rg2_off * 2, W * 2);
            L.want("mlp.router", &L.router, 0, (size_t)lc.experts * W * 2);
            for (int e = 0; e < lc.experts; e++) {
                const std::string p = "mlp.e" + std::to_string(e) + ".";
                L.want(p + "gate", &L.egu, (size_t)e * 2 * one, one);   // per expert: gate rows, then up rows
                L.want(p + "up", &L.egu, (size_t)e * 2 * one + one, one);
                L.want(p + "down", &L.edown, (size_t)e * one, one);
            }
            if (S) {
                GA(L.sdown, W * S * 2);
                L.want("mlp.shared.gate", &L.wfused2, (size_t)L.sgu_off * W * 2, S * W * 2);
                L.want("mlp.shared.up", &L.wfused2, (size_t)(L.sgu_off + S) * W * 2, S * W * 2);
                L.want("mlp.shared.sg", &L.wfused2, (size_t)L.sg_off * W * 2, W * 2);
                L.want("mlp.shared.down", &L.sdown, 0, W * S * 2);
            }
            ne = std::max(ne, (size_t)lc.experts);
            pairs = std::max(pairs, T * lc.top);
            cap = std::max(cap, T * lc.top + (size_t)lc.experts * 63);
            eff = std::max(eff, (size_t)lc.expert_ff);
            sff = std::max(sff, S);
            nf = std::max(nf, (size_t)L.nf2);
        } else if (ff) {
            vmx_set_error("gezozen_create: layer %d: unknown feed-forward kind %d", li, lc.mlp);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        nf = std::max(nf, (size_t)L.nf);
    }
#undef BAD
    GA(m->embed, (size_t)c.vocab * W * 2);
    GA(m->final_norm, W * 2);
    GA(m->head, (size_t)c.vocab * W * 2);
    m->missing = {"embed", "final.norm", "head"};
    GA(m->x, T * W * 4);
    GA(m->acc, T * W * 4);
    GA(m->h, T * W * m->esz());
    GA(m->hsel, T * W * m->esz());
    GA(m->fused, T * std::max(nf, (size_t)c.vocab) * 4);   // also the logits of a greedy-only step
    GA(m->qbuf, T * hd * 4);
    GA(m->attn, T * hv * m->esz());
    GA(m->attn_ws, attn_ws);   // key shares of attention launches with few rows
    GA(m->conv, T * convc * 4);
    GA(m->dec, T * rhd * 4);
    GA(m->dro, T * rhv * 4);
    GA(m->rec, T * rhv * m->esz());
    GA(m->argmax_keys, T * ((size_t)c.vocab / VMX_ARGMAX_CHUNK + 1) * 8);
    GA(m->few_pairs, (size_t)(2 * VMX_MOE_FEW_PAIRS * 16 + VMX_MOE_FEW_PAIRS + 1) * 4);
    GA(m->rlogits, T * ne * 4);
    GA(m->topw, (pairs + 1) * 4);
    GA(m->topi, (pairs + 1) * 4);
    GA(m->sorted, (cap + 1) * 4);
    GA(m->blk_expert, (cap / 16 + 2) * 4);
    GA(m->total, 16);
    GA(m->inv, (pairs + 1) * 4);
    GA(m->gu, (cap + 1) * 2 * eff * 4);
    GA(m->act, (cap + 1) * eff * m->esz());
    GA(m->ydown, (cap + 1) * W * 4);
    GA(m->sact, T * sff * m->esz());
    GA(m->sout, T * W * 4);
#undef GA
    if (!rc) {
        // decode steps with a handful of (token, slot) pairs skip the sort: pair p is its own 16-row block (row 16 p)
        const int FP = VMX_MOE_FEW_PAIRS;
        std::vector<int32_t> fp(2 * FP * 16 + FP + 1);
        for (int i = 0; i < FP * 16; i++) {
            fp[i] = i % 16 == 0 ? i / 16 : 0x7fffffff;              // gathered rows of the first product: pair index or padding
            fp[FP * 16 + i] = i % 16 == 0 ? i : 0x7fffffff;          // rows of the second product: themselves or padding
        }
        for (int p = 0; p < FP; p++) fp[2 * FP * 16 + p] = 16 * p;   // where pair p's result lies
        fp[2 * FP * 16 + FP] = 0x7fffffff;                           // "total rows": never cuts
        if (hipMemcpy(m->few_pairs.p, fp.data(), fp.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
            vmx_set_error("gezozen_create: upload failed");
            rc = VMX_ELAUNCH;
        }
    }
    if (rc) {
        vmx_gezozen_destroy(m);
        return rc;
    }
    *out = m;
    return VMX_OK;
}

extern "C" void vmx_gezozen_destroy(vmx_gezozen *m) {
    if (!m) return;
    for (Layer &L : m->layers)
        for (Buf *b : {&L.norm1, &L.norm2, &L.wfused, &L.bias, &L.wfused2, &L.bias2, &L.qnorm, &L.knorm, &L.wo, &L.rot_steps, &L.kcache, &L.vcache,
                       &L.wo_right, &L.onorm, &L.wa2, &L.a2b, &L.decay, &L.r_rot_steps, &L.s_state, &L.conv_taps, &L.a_log, &L.dt_bias, &L.conv_state,
                       &L.router, &L.egu, &L.edown, &L.sdown})
            b->release();
    for (Buf *b : {&m->embed, &m->final_norm, &m->head, &m->x, &m->acc, &m->h, &m->hsel, &m->fused, &m->qbuf, &m->attn, &m->attn_ws, &m->conv, &m->dec,
                   &m->dro, &m->rec, &m->argmax_keys, &m->few_pairs, &m->rlogits, &m->topw, &m->topi, &m->sorted, &m->blk_expert, &m->total, &m->inv,
                   &m->gu, &m->act, &m->ydown, &m->sact, &m->sout})
        b->release();
    delete m;
}

extern "C" int vmx_gezozen_load_tensor(vmx_gezozen *m, const char *name, const void *data, size_t bytes, void *stream) {
    VMX_REQUIRE(m && name && (data || bytes == 0), "gezozen_load_tensor: null pointer");
    hipStream_t st = vmx_stream(stream);
    const vmx_gezozen_config &c = m->cfg;
    const size_t W = c.width;
    const std::string n(name);
    Seg dst;
    std::vector<std::string> *missing = &m->missing;
    std::string key = n;
    if (n == "embed") dst = Seg{&m->embed, 0, (size_t)c.vocab * W * 2};
    else if (n == "final.norm") dst = Seg{&m->final_norm, 0, W * 2};
    else if (n == "head") dst = Seg{&m->head, 0, (size_t)c.vocab * W * 2};
    else if (n.size() > 1 && n[0] == 'l' && isdigit((unsigned char)n[1])) {
        const size_t dot = n.find('.');
        VMX_REQUIRE(dot != std::string::npos, "gezozen_load_tensor: unknown tensor `%s`", name);
        const int li = atoi(n.substr(1, dot - 1).c_str());
        VMX_REQUIRE(li >= 0 && li < c.num_layers, "gezozen_load_tensor: `%s`: the model has %d layers", name, c.num_layers);
        Layer &L = m->layers[li];
        missing = &L.missing;
        key = n.substr(dot + 1);
        for (const auto &t : L.tensors)
            if (t.first == key) dst = t.second;
    }
    VMX_REQUIRE(dst.buf, "gezozen_load_tensor: unknown tensor `%s`", name);
    VMX_REQUIRE(bytes == dst.bytes, "gezozen_load_tensor: `%s`: expected %zu bytes of bf16, got %zu", name, dst.bytes, bytes);
    if (bytes > 0)
        if (int rc = upload(*dst.buf, dst.offset, data, bytes, st)) return rc;
    erase_name(*missing, key);
    return VMX_OK;
}

extern "C" int vmx_gezozen_missing_tensors(const vmx_gezozen *m) {
    if (!m) return -1;
    size_t n = m->missing.size();
    std::string first = m->missing.empty() ? "" : m->missing[0];
    for (size_t li = 0; li < m->layers.size(); li++) {
        const Layer &L = m->layers[li];
        if (first.empty() && !L.missing.empty()) first = "l" + std::to_string(li) + "." + L.missing[0];
        n += L.missing.size();
    }
    if (n) vmx_set_error("gezozen: %zu tensors not loaded, first `%s`", n, first.c_str());
    return (int)n;
}

extern "C" int vmx_gezozen_forward(vmx_gezozen *m, const int32_t *tokens, const int32_t *positions, const int32_t *slots, const int32_t *seq_ids,
                                   int num_tokens, const int32_t *block_tables, int num_seqs, int max_blocks_per_seq, const int32_t *seq_starts,
                                   const int32_t *state_slots, const int32_t *logit_rows, int num_logit_rows, float *logits, int32_t *greedy_ids,
                                   float *layer_trace, void *stream) {
    VMX_REQUIRE(m && tokens && positions && slots && seq_ids && block_tables && seq_starts && state_slots, "gezozen_forward: null pointer");
    const vmx_gezozen_config &c = m->cfg;
    VMX_REQUIRE(num_tokens >= 1 && num_tokens <= c.max_tokens, "gezozen_forward: %d tokens, the model was created for at most %d", num_tokens,
                c.max_tokens);
    VMX_REQUIRE(num_seqs >= 1 && num_seqs <= c.max_seqs && max_blocks_per_seq >= 1, "gezozen_forward: bad sequence count or block-table shape");
    VMX_REQUIRE(num_logit_rows >= 0 && num_logit_rows <= num_tokens && (num_logit_rows == 0 || (logit_rows && (logits || greedy_ids))),
                "gezozen_forward: bad logit rows");
    if (vmx_gezozen_missing_tensors(m) != 0) return VMX_EINVAL;
    hipStream_t st = vmx_stream(stream);
    const int T = num_tokens, W = c.width, f32 = m->f32() ? 1 : 0;
    const int cdt = f32 ? VMX_F32 : VMX_BF16;
    float *x = m->x.as<float>(), *acc = m->acc.as<float>(), *fused = m->fused.as<float>();
    // acc = embed[token]; the norm kernel without gains turns it into x, its copy for the linears and alpha x
    if (int rc = vmx_embed_scaled_f32(acc, m->embed.as<uint16_t>(), tokens, T, W, c.vocab, 1.0f, st)) return rc;
    if (int rc = vmx_group_norm_post(acc, x, m->h.p, f32, nullptr, 1, W, c.norm_eps, c.postln_alpha, T, st)) return rc;
    for (int li = 0; li < c.num_layers; li++) {
        Layer &L = m->layers[li];
        const vmx_gezozen_layer_config &lc = L.c;
        const int nf = L.nf;
        {   // everything that reads the mixer's input
            VmxLinear p;
            p.A = m->h.p, p.a_f32 = f32, p.lda = W;
            p.W = L.wfused.as<uint16_t>(), p.w_sn = W, p.w_sk = 1, p.bias = L.bias.as<uint16_t>();
            p.C = fused, p.c_f32 = 1, p.ldc = nf;
            p.M = T, p.N = nf, p.K = W, p.exact = f32;
            if (int rc = vmx_linear_launch(p, st)) return rc;
        }
        const int RH = L.rh, RQ = L.rqk, RD = L.rd, RV = L.rv;
        float *dec = m->dec.as<float>(), *dro = m->dro.as<float>(), *cv = m->conv.as<float>();
        if (lc.mixer == VMX_MIXER_HEAD_DELTA) {
            const int H = lc.heads, G = lc.kv_heads, D = lc.dim, V = lc.vdim, C = 2 * G * D + H * V;
            if (int rc = vmx_short_conv_silu(fused + L.q_off, nf, L.conv_taps.as<uint16_t>(), L.conv_state.as<float>(), cv, C, positions, seq_ids,
                                             seq_starts, state_slots, T, C, lc.conv_taps, D, 2 * G, G, 1e-6f, 1.0f / sqrtf((float)D), st))
                return rc;
            if (int rc = vmx_short_conv_state_update(fused + L.q_off, nf, L.conv_state.as<float>(), positions, seq_starts, state_slots, num_seqs, C,
                                                     lc.conv_taps, st))
                return rc;
            // one decay per head: the gate kernel over "heads" of one channel
            if (int rc = vmx_delta_rule_gates(fused + L.a_off, nf, L.a_log.as<uint16_t>(), L.dt_bias.as<uint16_t>(), fused + L.b_off, nf, T, H, 1, st))
                return rc;
            if (int rc = vmx_matrix_memory_recurrence(dro, (int64_t)H * V, cv, C, 1.0f, cv + G * D, C, cv + 2 * G * D, C, fused + L.a_off, nf, 1,
                                                      fused + L.b_off, nf, L.s_state.as<float>(), positions, seq_starts, state_slots, num_seqs, H,
                                                      G, D, V, st))
                return rc;
        } else {
            const int H = lc.heads, G = lc.kv_heads, D = lc.dim, V = lc.vdim;
            vmx_qk_prepare_opts po = {1, 1, L.rot_mul, 1.0f, 1.0f, nullptr, 0};
            if (int rc = vmx_qk_prepare_ex(m->qbuf.as<float>(), fused + L.q_off, nf, H * D, fused + L.k_off, nf, G * D, fused + L.v_off, nf, G * V,
                                           L.qnorm.as<uint16_t>(), L.knorm.as<uint16_t>(), c.norm_eps, L.rot_steps.as<float>(), lc.rot.dims, D,
                                           positions, slots, L.kcache.p, L.vcache.p, cdt, T, &po, st))
                return rc;
            if (int rc = vmx_window_attention(m->attn.p, cdt, m->qbuf.as<float>(), (int64_t)H * D, L.kcache.p, L.vcache.p, cdt, block_tables,
                                              max_blocks_per_seq, seq_ids, positions, nullptr, nullptr, 0, lc.scale, lc.softcap, lc.window, 0, T, H, G,
                                              D, V, c.block_size, seq_starts, num_seqs, m->attn_ws.p, m->attn_ws.bytes, st))
                return rc;
            {   // acc += left_scale * sigmoid(gate 1) * W_o heads
                VmxLinear o;
                o.A = m->attn.p, o.a_f32 = f32, o.lda = (int64_t)H * V;
                o.W = L.wo.as<uint16_t>(), o.w_sn = (int64_t)H * V, o.w_sk = 1;
                o.C = acc, o.c_f32 = 1, o.ldc = W;
                o.M = T, o.N = W, o.K = H * V, o.exact = f32;
                o.epilogue = VMX_EP_ADD_MUL_SIGMOID, o.aux = fused + L.rg1_off, o.ldaux = nf, o.out_scale = lc.left_scale;
                if (int rc = vmx_linear_launch(o, st)) return rc;
            }
            if (lc.mixer == VMX_MIXER_ATTENTION_GLA) {
                VmxLinear a;   // decay logits: second half of the two-step projection, with its bias
                a.A = fused + L.a1_off, a.a_f32 = 1, a.lda = nf;
                a.W = L.wa2.as<uint16_t>(), a.w_sn = lc.decay_rank, a.w_sk = 1, a.bias = L.a2b.as<uint16_t>();
                a.C = dec, a.c_f32 = 1, a.ldc = (int64_t)RH * RD;
                a.M = T, a.N = RH * RD, a.K = lc.decay_rank, a.exact = f32;
                if (int rc = vmx_linear_launch(a, st)) return rc;
                if (int rc = vmx_sigmoid_root_decay(dec, (int64_t)RH * RD, T, RH * RD, lc.tau, st)) return rc;
                if (int rc = vmx_matrix_memory_recurrence(dro, (int64_t)RH * RV, fused + L.rq_off, nf, 1.0f / sqrtf((float)RD), fused + L.rk_off, nf,
                                                          fused + L.rv_off, nf, dec, (int64_t)RH * RD, 0, nullptr, 0, L.s_state.as<float>(),
                                                          positions, seq_starts, state_slots, num_seqs, RH, RQ, RD, RV, st))
                    return rc;
            } else {
                // q and k rotated into rows of their own (k also scaled); no cache: the memory carries the past
                float *rk = cv + (size_t)T * RH * RD;
                vmx_qk_prepare_opts ro = {1, 1, L.r_rot_mul, 1.0f, 1.0f / sqrtf((float)RD), rk, (int64_t)RH * RD};
                if (int rc = vmx_qk_prepare_ex(cv, fused + L.rq_off, nf, RH * RD, fused + L.rk_off, nf, RH * RD, nullptr, 0, 0, nullptr, nullptr,
                                               c.norm_eps, L.r_rot_steps.as<float>(), lc.r_rot.dims, RD, positions, nullptr, nullptr, nullptr, cdt, T,
                                               &ro, st))
                    return rc;
                if (int rc = vmx_matrix_memory_recurrence(dro, (int64_t)RH * RV, cv, (int64_t)RH * RD, 1.0f, rk, (int64_t)RH * RD, fused + L.rv_off, nf, L.decay.as<float>(), 0, 1, nullptr, 0, L.s_state.as<float>(), positions,
                                                          seq_starts, state_slots, num_seqs, RH, RQ, RD, RV, st))
                    return rc;
            }
        }
        // read-out: per-head RMS norm (gains where the mixer has them), times silu(W_g x)
        if (int rc = vmx_head_rms_gate_ex(m->rec.p, cdt, dro, (int64_t)RH * RV, L.onorm.p ? L.onorm.as<uint16_t>() : nullptr, fused + L.g_off, nf, 1,
                                          c.norm_eps, T, RH, RV, st))
            return rc;
        {   // acc += [right_scale *] sigmoid(gate 1) * W_o read-out
            VmxLinear o;
            o.A = m->rec.p, o.a_f32 = f32, o.lda = (int64_t)RH * RV;
            o.W = L.wo_right.as<uint16_t>(), o.w_sn = (int64_t)RH * RV, o.w_sk = 1;
            o.C = acc, o.c_f32 = 1, o.ldc = W;
            o.M = T, o.N = W, o.K = RH * RV, o.exact = f32;
            o.epilogue = VMX_EP_ADD_MUL_SIGMOID, o.aux = fused + L.rg1_off, o.ldaux = nf;
            o.out_scale = lc.mixer == VMX_MIXER_HEAD_DELTA ? 1.0f : lc.right_scale;
            if (int rc = vmx_linear_launch(o, st)) return rc;
        }
        if (int rc = vmx_group_norm_post(acc, x, m->h.p, f32, L.norm1.as<uint16_t>(), c.norm_groups, W, c.norm_eps, c.postln_alpha, T, st)) return rc;
        if (lc.mlp == VMX_MLP_SIGMOID_MOE) {
            const int E = lc.experts, k = lc.top, ff = lc.expert_ff, S = lc.shared_ff, nf2 = L.nf2, pairs = T * k, FP = VMX_MOE_FEW_PAIRS;
            {   // what reads the feed-forward's input besides the experts: shared gate | up, the shared expert's gate, residual gate 2
                VmxLinear p;
                p.A = m->h.p, p.a_f32 = f32, p.lda = W;
                p.W = L.wfused2.as<uint16_t>(), p.w_sn = W, p.w_sk = 1, p.bias = L.bias2.as<uint16_t>();
                p.C = fused, p.c_f32 = 1, p.ldc = nf2;
                p.M = T, p.N = nf2, p.K = W, p.exact = f32;
                if (int rc = vmx_linear_launch(p, st)) return rc;
            }
            VmxLinear r;   // router logits: always a true f32 product
            r.A = m->h.p, r.a_f32 = f32, r.lda = W;
            r.W = L.router.as<uint16_t>(), r.w_sn = W, r.w_sk = 1;
            r.C = m->rlogits.p, r.c_f32 = 1, r.ldc = E;
            r.M = T, r.N = E, r.K = W, r.exact = 1;
            if (int rc = vmx_linear_launch(r, st)) return rc;
            if (int rc = vmx_topk_sigmoid(m->rlogits.as<float>(), m->topw.as<float>(), m->topi.as<int32_t>(), T, E, k, 0, stream)) return rc;
            const bool few = pairs <= FP;   // every pair its own block: no sort
            const int br = few ? 16 : (pairs >= 32 * E ? 64 : 16);
            const int cap = few ? pairs * 16 : pairs + E * (br - 1);
            const int32_t *fp = m->few_pairs.as<int32_t>();
            const int32_t *up_rows = few ? fp : m->sorted.as<int32_t>(), *down_rows = few ? fp + FP * 16 : nullptr;
            const int32_t *blk = few ? m->topi.as<int32_t>() : m->blk_expert.as<int32_t>();
            const int32_t *total = few ? fp + 2 * FP * 16 + FP : m->total.as<int32_t>();
            const int32_t *inv = few ? fp + 2 * FP * 16 : m->inv.as<int32_t>();
            if (!few) {
                if (int rc = vmx_moe_align_block_size(m->topi.as<int32_t>(), m->sorted.as<int32_t>(), m->blk_expert.as<int32_t>(),
                                                      m->total.as<int32_t>(), pairs, E, br, cap, stream))
                    return rc;
                if (int rc = vmx_moe_inverse(m->inv.as<int32_t>(), m->sorted.as<int32_t>(), m->total.as<int32_t>(), pairs, cap, st)) return rc;
            }
            VmxLinear u;   // gate | up of the pairs' rows in one product
            u.A = m->h.p, u.a_f32 = f32, u.lda = W;
            u.W = L.egu.as<uint16_t>(), u.w_sn = W, u.w_sk = 1;
            u.C = m->gu.p, u.c_f32 = 1, u.ldc = 2 * ff;
            u.M = cap, u.N = 2 * ff, u.K = W, u.exact = f32;
            u.row_ids = up_rows, u.row_div = k, u.row_limit = pairs;
            u.block_expert = blk, u.expert_stride = (int64_t)2 * ff * W, u.block_rows = br, u.total_rows = total;
            if (int rc = vmx_linear_launch(u, st)) return rc;
            // the router's score scales the expert's input: silu(s g) * (s u), s = score of the row's pair
            if (int rc = vmx_glu_silu_rows_scaled(m->act.p, f32, m->gu.as<float>(), 2 * ff, ff, cap, ff, m->topw.as<float>(), up_rows, pairs, nullptr,
                                                  0, st))
                return rc;
            VmxLinear d;
            d.A = m->act.p, d.a_f32 = f32, d.lda = ff;
            d.W = L.edown.as<uint16_t>(), d.w_sn = ff, d.w_sk = 1;
            d.C = m->ydown.p, d.c_f32 = 1, d.ldc = W;
            d.M = cap, d.N = W, d.K = ff, d.exact = f32;
            d.row_ids = down_rows, d.row_div = 1, d.row_limit = cap;
            d.block_expert = blk, d.expert_stride = (int64_t)ff * W, d.block_rows = br, d.total_rows = total;
            if (int rc = vmx_linear_launch(d, st)) return rc;
            if (S) {   // shared expert: its per-token gate goes onto the rows of the down projection
                if (int rc = vmx_glu_silu_rows_scaled(m->sact.p, f32, fused + L.sgu_off, nf2, S, T, S, nullptr, nullptr, 0, fused + L.sg_off, nf2, st))
                    return rc;
                VmxLinear sd;
                sd.A = m->sact.p, sd.a_f32 = f32, sd.lda = S;
                sd.W = L.sdown.as<uint16_t>(), sd.w_sn = S, sd.w_sk = 1;
                sd.C = m->sout.p, sd.c_f32 = 1, sd.ldc = W;
                sd.M = T, sd.N = W, sd.K = S, sd.exact = f32;
                if (int rc = vmx_linear_launch(sd, st)) return rc;
            }
            if (int rc = vmx_moe_combine_f32(acc, m->ydown.as<float>(), inv, nullptr, k, S ? m->sout.as<float>() : nullptr, fused + L.rg2_off, nf2, T,
                                             W, st))
                return rc;
            if (int rc = vmx_group_norm_post(acc, x, m->h.p, f32, L.norm2.as<uint16_t>(), c.norm_groups, W, c.norm_eps, c.postln_alpha, T, st)) return rc;
        }
        if (layer_trace)
            VMX_CHECK_HIP(hipMemcpyAsync(layer_trace + (size_t)li * T * W, x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    }
    if (num_logit_rows > 0) {
        if (int rc = vmx_group_norm_rows(m->hsel.p, f32, x, logit_rows, m->final_norm.as<uint16_t>(), c.norm_groups, W, c.norm_eps, num_logit_rows, st))
            return rc;
        float *lg = logits ? logits : fused;   // greedy ids only: the logits live in a workspace
        VmxLinear hd;
        hd.A = m->hsel.p, hd.a_f32 = f32, hd.lda = W;
        hd.W = m->head.as<uint16_t>(), hd.w_sn = W, hd.w_sk = 1;
        hd.C = lg, hd.c_f32 = 1, hd.ldc = c.vocab;
        hd.M = num_logit_rows, hd.N = c.vocab, hd.K = W, hd.exact = f32;
        if (int rc = vmx_linear_launch(hd, st)) return rc;
        if (greedy_ids)
            if (int rc = vmx_argmax_f32_rows(greedy_ids, m->argmax_keys.as<unsigned long long>(), lg, num_logit_rows, c.vocab, st)) return rc;
    }
    return VMX_OK;
}
