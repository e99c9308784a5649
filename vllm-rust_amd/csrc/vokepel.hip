// Whole-step executor of the Vokepel decoder family: pre-norm layers listed in the model's configuration,
//   x += m * mixer(norm1(x));   x += m * ff(norm2(x))                  (one multiplier m for the model; ff may be absent)
//   logits = cap * tanh(embed . norm(x) * logit_scale / cap)            (the embedding table is the output matrix)
// A run of layers [start, stop) may LOOP: it runs `times` times in a row with the same weights, every pass starting from
// x <- W_in [x | x0] + step[pass] (x0 = the embedding output).  Every (layer, pass) is a LAYER RUN with a key/value cache and a
// recurrent state of its own.
// Mixer "attention" (VMX_MIXER_TALKING_ATTENTION): grouped-query attention whose values are the keys as projected; q and k are
// RMS-normed over their whole rows; scores are scaled, soft-capped, reduced by r1 ln(1 + r2 (i - j)) and mixed across the heads
// before the softmax over a sliding window; the concatenated heads are gated element-wise by sigmoid(W_g h).
// Mixer "parallel" (VMX_MIXER_ATTENTION_GRU): left_scale * (grouped-query attention with interleaved-pair rotation of the first
// rot_dims coordinates of every head, a sliding window and a learned sink in the softmax denominator) + right_scale * (a minimal
// gated recurrent unit, min_gru.hip, with a SiLU output gate); both read the same h and have output matrices of their own.
// Feed-forward: W_down relu(W_up h)^2.
//
// Every product that reads h (q, k, [v,] gates, recurrent-unit inputs) is ONE linear whose f32 output row the other kernels address
// by column offset.  The residual stream, norms, positions and angles, scores, softmax, the recurrence and its state are f32 in
// both modes; VMX_BF16 rounds the operands of the linears and the cache rows to bf16, VMX_F32 multiplies in true f32 everywhere.
// The forward call allocates nothing, reads nothing back and is graph-capturable.
#include "vmx_kernels.h"
#include <math.h>
#include <algorithm>
#include <string>
#include <vector>

namespace {

using Buf = VmxBuf;

int pad8(int n) { return (n + 7) & ~7; }

struct Seg {       // where a checkpoint tensor lands: rows of the fused projection, or a buffer of its own
    Buf *buf = nullptr;
    size_t offset = 0, bytes = 0;
};

struct Layer {
    vmx_vokepel_layer_config c;
    Buf norm1, norm2, wfused, bias, wo, wo_right, qnorm, knorm, r1, r2, talk, sink, inv_freq, wup, wdown;
    int nf = 0, q_off = 0, k_off = 0, v_off = 0, g_off = 0, z_off = 0, u_off = 0;
    int vdim = 0;   // value size of the attention as it runs (the talking attention's values are its keys)
    std::vector<std::pair<std::string, Seg>> tensors;
    std::vector<std::string> missing;
    void want(const std::string &name, Buf *b, size_t off, size_t bytes) {
        tensors.push_back({name, Seg{b, off, bytes}});
        missing.push_back(name);
    }
};

struct Run {       // one execution of a layer: its own cache and state
    int layer = 0, pass = -1;   // pass >= 0: inside the loop; the first layer of a pass is preceded by the loop's input step
    bool enters_pass = false;
    Buf kcache, vcache, gru_state;
};

}  // namespace

struct vmx_vokepel {
    vmx_vokepel_config cfg;
    std::vector<Layer> layers;
    std::vector<Run> runs;
    Buf embed, final_norm, loop_in, loop_step;
    std::vector<std::string> missing;
    Buf x, x0, cat, h, hsel, fused, qbuf, attn, attn_ws, gru, act, argmax_keys;
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

}  // namespace

extern "C" int vmx_vokepel_create(const vmx_vokepel_config *cfg, const vmx_vokepel_layer_config *layer_cfgs, vmx_vokepel **out) {
    VMX_REQUIRE(cfg && layer_cfgs && out, "vokepel_create: null pointer");
    const vmx_vokepel_config &c = *cfg;
    VMX_REQUIRE(c.vocab >= 1 && c.width >= 1 && c.num_layers >= 1, "vokepel_create: bad sizes (vocab %d, width %d, layers %d)", c.vocab, c.width,
                c.num_layers);
    VMX_REQUIRE(c.dtype == VMX_F32 || c.dtype == VMX_BF16, "vokepel_create: dtype must be VMX_F32 or VMX_BF16");
    VMX_REQUIRE(c.block_size >= 1 && c.num_blocks >= 1 && c.max_tokens >= 1 && c.max_seqs >= 1 && c.state_slots >= 1,
                "vokepel_create: bad cache / batch geometry");
    VMX_REQUIRE(c.loop_times >= 0 && (c.loop_times == 0 || (c.loop_start >= 0 && c.loop_start < c.loop_stop && c.loop_stop <= c.num_layers)),
                "vokepel_create: the loop [%d, %d) x %d does not lie inside %d layers", c.loop_start, c.loop_stop, c.loop_times, c.num_layers);
    VMX_REQUIRE(c.logit_softcap >= 0.f, "vokepel_create: negative logit soft cap");
    vmx_vokepel *m = new vmx_vokepel();
    m->cfg = c;
    m->layers.resize(c.num_layers);
    const size_t T = c.max_tokens, W = c.width, rows = (size_t)c.num_blocks * c.block_size;
    size_t attn_ws = 16, nf = 8, hv = 1, hd = 1, gw = 1, actn = 1;
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
        const vmx_vokepel_layer_config &lc = L.c;
        if (lc.heads < 1 || lc.kv_heads < 1 || lc.heads % lc.kv_heads || lc.dim < 1 || lc.dim > 256 || lc.vdim < 1 || lc.vdim > 256)
            BAD("vokepel_create: layer %d: bad head counts or sizes (heads %d, kv_heads %d, dim %d, vdim %d; sizes up to 256)", li, lc.heads,
                lc.kv_heads, lc.dim, lc.vdim);
        if (lc.window < 0 || lc.softcap < 0.f) BAD("vokepel_create: layer %d: bad attention mask or soft cap", li);
        const size_t H = lc.heads, G = lc.kv_heads, D = lc.dim;
        int at = 0;
        auto seg = [&](int n) {
            const int o = at;
            at = pad8(at + n);
            return o;
        };
        L.want("norm1", &L.norm1, 0, W * 2);
        GA(L.norm1, W * 2);
        if (lc.mixer == VMX_MIXER_TALKING_ATTENTION) {
            if (lc.vdim != lc.dim) BAD("vokepel_create: layer %d: the values of this attention are its keys, vdim %d != dim %d", li, lc.vdim, lc.dim);
            if (lc.heads > 64 || H * D > 8192) BAD("vokepel_create: layer %d: mixed heads take at most 64 heads and 8192 query numbers per token", li);
            L.vdim = lc.dim;
            L.q_off = seg(H * D);
            L.k_off = seg(G * D);
            L.g_off = seg(H * D);
            L.nf = at;
            GA(L.wfused, (size_t)L.nf * W * 2);
            GA(L.wo, W * H * D * 2);
            GA(L.qnorm, H * D * 2);
            GA(L.knorm, G * D * 2);
            GA(L.r1, H * 2);
            GA(L.r2, H * 2);
            GA(L.talk, H * H * 2);
            L.want("mix.q", &L.wfused, (size_t)L.q_off * W * 2, H * D * W * 2);
            L.want("mix.k", &L.wfused, (size_t)L.k_off * W * 2, G * D * W * 2);
            L.want("mix.g", &L.wfused, (size_t)L.g_off * W * 2, H * D * W * 2);
            L.want("mix.q.norm", &L.qnorm, 0, H * D * 2);
            L.want("mix.k.norm", &L.knorm, 0, G * D * 2);
            L.want("mix.r1", &L.r1, 0, H * 2);
            L.want("mix.r2", &L.r2, 0, H * 2);
            L.want("mix.talk", &L.talk, 0, H * H * 2);
            L.want("mix.o", &L.wo, 0, W * H * D * 2);
        } else if (lc.mixer == VMX_MIXER_ATTENTION_GRU) {
            if (lc.gru_width < 1) BAD("vokepel_create: layer %d: bad recurrent width %d", li, lc.gru_width);
            if (lc.rot_dims < 0 || lc.rot_dims > lc.dim || lc.rot_dims % 2 || (lc.rot_dims > 0 && (lc.dim % 2 || !(lc.rot_base > 0.0))))
                BAD("vokepel_create: layer %d: %d rotated coordinates (base %g) in heads of %d", li, lc.rot_dims, lc.rot_base, lc.dim);
            const size_t V = lc.vdim, R = lc.gru_width;
            L.vdim = lc.vdim;
            L.q_off = seg(H * D);
            L.k_off = seg(G * D);
            L.v_off = seg(G * V);
            L.z_off = seg(R);
            L.u_off = seg(R);
            L.g_off = seg(R);
            L.nf = at;
            GA(L.wfused, (size_t)L.nf * W * 2);
            GA(L.bias, (size_t)L.nf * 2);
            GA(L.wo, W * H * V * 2);
            GA(L.wo_right, W * R * 2);
            GA(L.sink, H * 2);
            L.want("mix.left.q", &L.wfused, (size_t)L.q_off * W * 2, H * D * W * 2);
            L.want("mix.left.k", &L.wfused, (size_t)L.k_off * W * 2, G * D * W * 2);
            L.want("mix.left.v", &L.wfused, (size_t)L.v_off * W * 2, G * V * W * 2);
            L.want("mix.left.sink", &L.sink, 0, H * 2);
            L.want("mix.left.o", &L.wo, 0, W * H * V * 2);
            L.want("mix.right.z", &L.wfused, (size_t)L.z_off * W * 2, R * W * 2);
            L.want("mix.right.z.b", &L.bias, (size_t)L.z_off * 2, R * 2);
            L.want("mix.right.x", &L.wfused, (size_t)L.u_off * W * 2, R * W * 2);
            L.want("mix.right.x.b", &L.bias, (size_t)L.u_off * 2, R * 2);
            L.want("mix.right.g", &L.wfused, (size_t)L.g_off * W * 2, R * W * 2);
            L.want("mix.right.o", &L.wo_right, 0, W * R * 2);
            if (lc.rot_dims > 0 && !rc) {   // angle steps per pair: base^(-2 i / dims), rounded once from double
                std::vector<float> f(lc.rot_dims / 2);
                for (int i = 0; i < lc.rot_dims / 2; i++) f[i] = (float)pow(lc.rot_base, -2.0 * i / lc.rot_dims);
                GA(L.inv_freq, f.size() * 4);
                if (!rc && hipMemcpy(L.inv_freq.p, f.data(), f.size() * 4, hipMemcpyHostToDevice) != hipSuccess) BAD("vokepel_create: upload failed");
            }
            gw = std::max(gw, R);
        } else {
            vmx_set_error("vokepel_create: layer %d: unknown mixer kind %d", li, lc.mixer);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        attn_ws = std::max(attn_ws, vmx_window_attention_workspace_bytes((int)T, lc.heads, L.vdim));
        if (lc.mlp == VMX_MLP_DENSE_RELU2) {
            if (lc.ff < 1) BAD("vokepel_create: layer %d: bad feed-forward width", li);
            GA(L.norm2, W * 2);
            GA(L.wup, (size_t)lc.ff * W * 2);
            GA(L.wdown, (size_t)lc.ff * W * 2);
            L.want("norm2", &L.norm2, 0, W * 2);
            L.want("mlp.up", &L.wup, 0, (size_t)lc.ff * W * 2);
            L.want("mlp.down", &L.wdown, 0, (size_t)lc.ff * W * 2);
            actn = std::max(actn, T * lc.ff);
        } else if (lc.mlp != VMX_MLP_NONE) {
            vmx_set_error("vokepel_create: layer %d: unknown feed-forward kind %d", li, lc.mlp);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        nf = std::max(nf, (size_t)L.nf);
        hv = std::max(hv, H * (size_t)L.vdim);
        hd = std::max(hd, H * D);
    }
#undef BAD
    // the order in which layers run; a looped layer once per pass
    if (!rc) {
        auto add = [&](int li, int pass, bool enters) {
            Run r;
            r.layer = li, r.pass = pass, r.enters_pass = enters;
            m->runs.push_back(r);
        };
        const int a = c.loop_times > 0 ? c.loop_start : c.num_layers, b = c.loop_times > 0 ? c.loop_stop : c.num_layers;
        for (int li = 0; li < a; li++) add(li, -1, false);
        for (int t = 0; t < c.loop_times; t++)
            for (int li = a; li < b; li++) add(li, t, li == a);
        for (int li = b; li < c.num_layers; li++) add(li, -1, false);
        for (Run &r : m->runs) {
            const Layer &L = m->layers[r.layer];
            GA(r.kcache, rows * L.c.kv_heads * L.c.dim * m->esz());
            GA(r.vcache, rows * L.c.kv_heads * L.vdim * m->esz());
            if (L.c.mixer == VMX_MIXER_ATTENTION_GRU) GA(r.gru_state, vmx_min_gru_state_bytes(c.state_slots, L.c.gru_width));
        }
    }
    GA(m->embed, (size_t)c.vocab * W * 2);
    GA(m->final_norm, W * 2);
    m->missing = {"embed", "final.norm"};
    if (c.loop_times > 0) {
        GA(m->loop_in, 2 * W * W * 2);
        GA(m->loop_step, (size_t)c.loop_times * W * 2);
        GA(m->x0, T * W * 4);
        GA(m->cat, T * 2 * W * m->esz());
        m->missing.push_back("loop.in");
        m->missing.push_back("loop.step");
    }
    GA(m->x, T * W * 4);
    GA(m->h, T * W * m->esz());
    GA(m->hsel, T * W * m->esz());
    GA(m->fused, T * std::max(nf, (size_t)c.vocab) * 4);   // also the logits of a greedy-only step
    GA(m->qbuf, T * hd * 4);
    GA(m->attn, T * hv * m->esz());
    GA(m->attn_ws, attn_ws);
    GA(m->gru, T * gw * m->esz());
    GA(m->act, actn * m->esz());
    GA(m->argmax_keys, T * ((size_t)c.vocab / VMX_ARGMAX_CHUNK + 1) * 8);
#undef GA
    if (rc) {
        vmx_vokepel_destroy(m);
        return rc;
    }
    *out = m;
    return VMX_OK;
}

extern "C" void vmx_vokepel_destroy(vmx_vokepel *m) {
    if (!m) return;
    for (Layer &L : m->layers)
        for (Buf *b : {&L.norm1, &L.norm2, &L.wfused, &L.bias, &L.wo, &L.wo_right, &L.qnorm, &L.knorm, &L.r1, &L.r2, &L.talk, &L.sink, &L.inv_freq,
                       &L.wup, &L.wdown})
            b->release();
    for (Run &r : m->runs)
        for (Buf *b : {&r.kcache, &r.vcache, &r.gru_state}) b->release();
    for (Buf *b : {&m->embed, &m->final_norm, &m->loop_in, &m->loop_step, &m->x, &m->x0, &m->cat, &m->h, &m->hsel, &m->fused, &m->qbuf, &m->attn,
                   &m->attn_ws, &m->gru, &m->act, &m->argmax_keys})
        b->release();
    delete m;
}

extern "C" int vmx_vokepel_num_layer_runs(const vmx_vokepel *m) { return m ? (int)m->runs.size() : 0; }

extern "C" int vmx_vokepel_load_tensor(vmx_vokepel *m, const char *name, const void *data, size_t bytes, void *stream) {
    VMX_REQUIRE(m && name && (data || bytes == 0), "vokepel_load_tensor: null pointer");
    hipStream_t st = vmx_stream(stream);
    const vmx_vokepel_config &c = m->cfg;
    const size_t W = c.width;
    const std::string n(name);
    Seg dst;
    std::vector<std::string> *missing = &m->missing;
    std::string key = n;
    if (n == "embed") dst = Seg{&m->embed, 0, (size_t)c.vocab * W * 2};
    else if (n == "final.norm") dst = Seg{&m->final_norm, 0, W * 2};
    else if (n == "loop.in" && c.loop_times > 0) dst = Seg{&m->loop_in, 0, 2 * W * W * 2};
    else if (n == "loop.step" && c.loop_times > 0) dst = Seg{&m->loop_step, 0, (size_t)c.loop_times * W * 2};
    else if (n.size() > 1 && n[0] == 'l' && isdigit((unsigned char)n[1])) {
        const size_t dot = n.find('.');
        VMX_REQUIRE(dot != std::string::npos, "vokepel_load_tensor: unknown tensor `%s`", name);
        const int li = atoi(n.substr(1, dot - 1).c_str());
        VMX_REQUIRE(li >= 0 && li < c.num_layers, "vokepel_load_tensor: `%s`: the model has %d layers", name, c.num_layers);
        Layer &L = m->layers[li];
        missing = &L.missing;
        key = n.substr(dot + 1);
        for (const auto &t : L.tensors)
            if (t.first == key) dst = t.second;
    }
    VMX_REQUIRE(dst.buf, "vokepel_load_tensor: unknown tensor `%s`", name);
    VMX_REQUIRE(bytes == dst.bytes, "vokepel_load_tensor: `%s`: expected %zu bytes of bf16, got %zu", name, dst.bytes, bytes);
    if (bytes > 0)
        if (int rc = upload(*dst.buf, dst.offset, data, bytes, st)) return rc;
    erase_name(*missing, key);
    return VMX_OK;
}

extern "C" int vmx_vokepel_missing_tensors(const vmx_vokepel *m) {
    if (!m) return -1;
    size_t n = m->missing.size();
    std::string first = m->missing.empty() ? "" : m->missing[0];
    for (size_t li = 0; li < m->layers.size(); li++) {
        const Layer &L = m->layers[li];
        if (first.empty() && !L.missing.empty()) first = "l" + std::to_string(li) + "." + L.missing[0];
        n += L.missing.size();
    }
    if (n) vmx_set_error("vokepel: %zu tensors not loaded, first `%s`", n, first.c_str());
    return (int)n;
}

extern "C" int vmx_vokepel_forward(vmx_vokepel *m, const int32_t *tokens, const int32_t *positions, const int32_t *slots, const int32_t *seq_ids,
                                   int num_tokens, const int32_t *block_tables, int num_seqs, int max_blocks_per_seq, const int32_t *seq_starts,
                                   const int32_t *state_slots, const int32_t *logit_rows, int num_logit_rows, float *logits, int32_t *greedy_ids,
                                   float *layer_trace, void *stream) {
    VMX_REQUIRE(m && tokens && positions && slots && seq_ids && block_tables && seq_starts && state_slots, "vokepel_forward: null pointer");
    const vmx_vokepel_config &c = m->cfg;
    VMX_REQUIRE(num_tokens >= 1 && num_tokens <= c.max_tokens, "vokepel_forward: %d tokens, the model was created for at most %d", num_tokens,
                c.max_tokens);
    VMX_REQUIRE(num_seqs >= 1 && num_seqs <= c.max_seqs && max_blocks_per_seq >= 1, "vokepel_forward: bad sequence count or block-table shape");
    VMX_REQUIRE(num_logit_rows >= 0 && num_logit_rows <= num_tokens && (num_logit_rows == 0 || (logit_rows && (logits || greedy_ids))),
                "vokepel_forward: bad logit rows");
    if (vmx_vokepel_missing_tensors(m) != 0) return VMX_EINVAL;
    hipStream_t st = vmx_stream(stream);
    const int T = num_tokens, W = c.width, f32 = m->f32() ? 1 : 0;
    const int cdt = f32 ? VMX_F32 : VMX_BF16;
    const float mult = c.residual_mult;
    float *x = m->x.as<float>(), *fused = m->fused.as<float>(), *qb = m->qbuf.as<float>();
    const bool looped = c.loop_times > 0;
    if (int rc = vmx_embed_scaled_f32(x, m->embed.as<uint16_t>(), tokens, T, W, c.vocab, 1.0f, st)) return rc;
    if (looped) VMX_CHECK_HIP(hipMemcpyAsync(m->x0.p, x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    for (size_t ri = 0; ri < m->runs.size(); ri++) {
        Run &R = m->runs[ri];
        Layer &L = m->layers[R.layer];
        const vmx_vokepel_layer_config &lc = L.c;
        const int H = lc.heads, G = lc.kv_heads, D = lc.dim, V = L.vdim, nf = L.nf;
        if (R.enters_pass) {   // x <- W_in [x | x0] + step[pass]
            if (int rc = vmx_concat2_rows(m->cat.p, f32, x, m->x0.as<float>(), T, W, st)) return rc;
            VmxLinear p;
            p.A = m->cat.p, p.a_f32 = f32, p.lda = 2 * W;
            p.W = m->loop_in.as<uint16_t>(), p.w_sn = 2 * W, p.w_sk = 1, p.bias = m->loop_step.as<uint16_t>() + (size_t)R.pass * W;
            p.C = x, p.c_f32 = 1, p.ldc = W;
            p.M = T, p.N = W, p.K = 2 * W, p.exact = f32;
            if (int rc = vmx_linear_launch(p, st)) return rc;
        }
        if (int rc = vmx_rms_norm_f32in(m->h.p, f32, x, nullptr, L.norm1.as<uint16_t>(), 0, W, c.norm_eps, T, st)) return rc;
        {   // everything that reads h
            VmxLinear p;
            p.A = m->h.p, p.a_f32 = f32, p.lda = W;
            p.W = L.wfused.as<uint16_t>(), p.w_sn = W, p.w_sk = 1, p.bias = L.bias.p ? L.bias.as<uint16_t>() : nullptr;
            p.C = fused, p.c_f32 = 1, p.ldc = nf;
            p.M = T, p.N = nf, p.K = W, p.exact = f32;
            if (int rc = vmx_linear_launch(p, st)) return rc;
        }
        vmx_window_attn_extras ex = {nullptr, nullptr, nullptr, nullptr, 0};
        if (lc.mixer == VMX_MIXER_TALKING_ATTENTION) {
            // keys normed over the whole row into the key cache, the same rows un-normed into the value cache
            if (int rc = vmx_qk_prepare_cache_write(qb, fused + L.q_off, nf, H * D, fused + L.k_off, nf, G * D, fused + L.k_off, nf, G * D,
                                                    L.qnorm.as<uint16_t>(), L.knorm.as<uint16_t>(), c.norm_eps, nullptr, 0, D, positions, slots,
                                                    R.kcache.p, R.vcache.p, cdt, T, st))
                return rc;
            ex.dist_r1_bf16 = L.r1.as<uint16_t>(), ex.dist_r2_bf16 = L.r2.as<uint16_t>(), ex.talk_bf16 = L.talk.as<uint16_t>();
            ex.gate_per_element = 1;
            if (int rc = vmx_window_attention_ex(m->attn.p, cdt, qb, (int64_t)H * D, R.kcache.p, R.vcache.p, cdt, block_tables, max_blocks_per_seq,
                                                 seq_ids, positions, nullptr, fused + L.g_off, nf, lc.scale, lc.softcap, lc.window, 0, T, H, G, D, V,
                                                 c.block_size, seq_starts, num_seqs, m->attn_ws.p, m->attn_ws.bytes, &ex, st))
                return rc;
        } else {
            if (int rc = vmx_qk_prepare_cache_write(qb, fused + L.q_off, nf, H * D, fused + L.k_off, nf, G * D, fused + L.v_off, nf, G * V, nullptr,
                                                    nullptr, c.norm_eps, L.inv_freq.as<float>(), lc.rot_dims, D, positions, slots, R.kcache.p,
                                                    R.vcache.p, cdt, T, st))
                return rc;
            ex.sink_bf16 = L.sink.as<uint16_t>();
            if (int rc = vmx_window_attention_ex(m->attn.p, cdt, qb, (int64_t)H * D, R.kcache.p, R.vcache.p, cdt, block_tables, max_blocks_per_seq,
                                                 seq_ids, positions, nullptr, nullptr, 0, lc.scale, 0.f, lc.window, 0, T, H, G, D, V, c.block_size,
                                                 seq_starts, num_seqs, m->attn_ws.p, m->attn_ws.bytes, &ex, st))
                return rc;
            if (int rc = vmx_min_gru(m->gru.p, cdt, fused + L.z_off, nf, fused + L.u_off, nf, fused + L.g_off, nf, R.gru_state.as<float>(), positions,
                                     seq_starts, state_slots, num_seqs, T, lc.gru_width, st))
                return rc;
            VmxLinear r;   // x += m * right_scale * W_o (S * silu(gate))
            r.A = m->gru.p, r.a_f32 = f32, r.lda = lc.gru_width;
            r.W = L.wo_right.as<uint16_t>(), r.w_sn = lc.gru_width, r.w_sk = 1;
            r.C = x, r.c_f32 = 1, r.ldc = W;
            r.M = T, r.N = W, r.K = lc.gru_width, r.exact = f32;
            r.epilogue = VMX_EP_ADD_F32, r.out_scale = mult * lc.right_scale;
            if (int rc = vmx_linear_launch(r, st)) return rc;
        }
        {   // x += m [* left_scale] * W_o heads
            VmxLinear o;
            o.A = m->attn.p, o.a_f32 = f32, o.lda = (int64_t)H * V;
            o.W = L.wo.as<uint16_t>(), o.w_sn = (int64_t)H * V, o.w_sk = 1;
            o.C = x, o.c_f32 = 1, o.ldc = W;
            o.M = T, o.N = W, o.K = H * V, o.exact = f32;
            o.epilogue = VMX_EP_ADD_F32, o.out_scale = lc.mixer == VMX_MIXER_ATTENTION_GRU ? mult * lc.left_scale : mult;
            if (int rc = vmx_linear_launch(o, st)) return rc;
        }
        if (lc.mlp == VMX_MLP_DENSE_RELU2) {
            if (int rc = vmx_rms_norm_f32in(m->h.p, f32, x, nullptr, L.norm2.as<uint16_t>(), 0, W, c.norm_eps, T, st)) return rc;
            VmxLinear u;
            u.A = m->h.p, u.a_f32 = f32, u.lda = W;
            u.W = L.wup.as<uint16_t>(), u.w_sn = W, u.w_sk = 1;
            u.C = m->act.p, u.c_f32 = f32, u.ldc = lc.ff;
            u.M = T, u.N = lc.ff, u.K = W, u.exact = f32, u.epilogue = VMX_EP_RELU2;
            if (int rc = vmx_linear_launch(u, st)) return rc;
            VmxLinear d;
            d.A = m->act.p, d.a_f32 = f32, d.lda = lc.ff;
            d.W = L.wdown.as<uint16_t>(), d.w_sn = lc.ff, d.w_sk = 1;
            d.C = x, d.c_f32 = 1, d.ldc = W;
            d.M = T, d.N = W, d.K = lc.ff, d.exact = f32;
            d.epilogue = VMX_EP_ADD_F32, d.out_scale = mult;
            if (int rc = vmx_linear_launch(d, st)) return rc;
        }
        if (layer_trace) VMX_CHECK_HIP(hipMemcpyAsync(layer_trace + ri * (size_t)T * W, x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    }
    if (num_logit_rows > 0) {
        if (int rc = vmx_rms_norm_f32in(m->hsel.p, f32, x, logit_rows, m->final_norm.as<uint16_t>(), 0, W, c.norm_eps, num_logit_rows, st)) return rc;
        float *lg = logits ? logits : fused;   // greedy ids only: the logits live in a workspace
        VmxLinear hd;
        hd.A = m->hsel.p, hd.a_f32 = f32, hd.lda = W;
        hd.W = m->embed.as<uint16_t>(), hd.w_sn = W, hd.w_sk = 1;
        hd.C = lg, hd.c_f32 = 1, hd.ldc = c.vocab;
        hd.M = num_logit_rows, hd.N = c.vocab, hd.K = W, hd.exact = f32;
        if (int rc = vmx_linear_launch(hd, st)) return rc;
        if (int rc = vmx_scale_softcap_f32(lg, (int64_t)num_logit_rows * c.vocab, c.logit_scale, c.logit_softcap, st)) return rc;
        if (greedy_ids)
            if (int rc = vmx_argmax_f32_rows(greedy_ids, m->argmax_keys.as<unsigned long long>(), lg, num_logit_rows, c.vocab, st)) return rc;
    }
    return VMX_OK;
}
