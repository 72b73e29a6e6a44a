"""The llama graph restatement (ug_amd/csrc/host/llama.cpp, after ug-llama/src/model.rs) against an
independent float64 numpy implementation of the same architecture, on the CPU oracle device.

No reference fixture holds llama outputs, so this is what pins the graph builders: RMSNorm, GQA
attention with rotary embeddings (both layouts) and a KV cache, SwiGLU, tied output head, written
from the textbook definitions rather than from the lazy-buffer code.  Greedy ids must agree and the
top-1 logit margins must agree to 1e-3 relative (f32 model vs f64 reference)."""
import ctypes as C

import numpy as np
import pytest

import ug_amd
from ug_amd import rng

SEED, STD = 9, 0.3


def weight(name, *shape):
    n = int(np.prod(shape))
    out = np.zeros(n, np.float32)
    assert ug_amd.host_lib().ugh_synthetic_weights(C.c_uint64(SEED), C.c_float(STD), 0, name.encode(), C.c_size_t(n), out.ctypes.data_as(C.c_void_p)) == 0
    return out.reshape(shape).astype(np.float64)


class NumpyLlama:
    def __init__(self, cfg, norm_mean=0.0):
        self.cfg = cfg
        h, isz = cfg.hidden_size, cfg.intermediate_size
        self.nh, self.nkv, self.hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        kv = self.nkv * self.hd
        self.embed = weight("model.embed_tokens.weight", cfg.vocab_size, h)
        def norm_w(name):   # norm vectors are norm_mean + N(0, std), summed in f32 like the generator does
            return (np.float32(norm_mean) + weight(name, h).astype(np.float32)).astype(np.float64)
        self.norm = norm_w("model.norm.weight")
        self.layers = []
        for i in range(cfg.num_hidden_layers):
            p = f"model.layers.{i}"
            self.layers.append(dict(
                rms1=norm_w(p + ".input_layernorm.weight"), rms2=norm_w(p + ".post_attention_layernorm.weight"),
                gate=weight(p + ".mlp.gate_proj.weight", isz, h), up=weight(p + ".mlp.up_proj.weight", isz, h), down=weight(p + ".mlp.down_proj.weight", h, isz),
                q=weight(p + ".self_attn.q_proj.weight", h, h), k=weight(p + ".self_attn.k_proj.weight", kv, h),
                v=weight(p + ".self_attn.v_proj.weight", kv, h), o=weight(p + ".self_attn.o_proj.weight", h, h)))
        # inverse frequencies are computed in f32 by the model (model.rs:277-284); angles in f64 here
        inv = np.array([np.float32(1.0) / np.float32(cfg.rope_theta) ** (np.float32(i) / np.float32(self.hd)) for i in range(0, self.hd, 2)], np.float32)
        self.inv_freq = inv.astype(np.float64)
        self.cache = [(np.zeros((self.nkv, 0, self.hd)), np.zeros((self.nkv, 0, self.hd))) for _ in self.layers]

    def rms(self, x, w):
        return x / np.sqrt((x * x).mean(-1, keepdims=True) + self.cfg.rms_norm_eps) * w

    def rotate(self, x, pos0):
        """x: [heads, t, hd]."""
        t = x.shape[1]
        ang = (pos0 + np.arange(t))[:, None] * self.inv_freq[None, :]   # [t, hd/2]
        c, s = np.cos(ang), np.sin(ang)
        out = np.empty_like(x)
        if self.cfg.rope_interleaved:
            a, b = x[..., 0::2], x[..., 1::2]
            out[..., 0::2], out[..., 1::2] = a * c - b * s, a * s + b * c
        else:
            half = self.hd // 2
            a, b = x[..., :half], x[..., half:]
            out[..., :half], out[..., half:] = a * c - b * s, a * s + b * c
        return out

    def forward(self, ids, pos0):
        x = self.embed[np.asarray(ids)]                                 # [t, h]
        t = x.shape[0]
        for li, l in enumerate(self.layers):
            hn = self.rms(x, l["rms1"])
            q = (hn @ l["q"].T).reshape(t, self.nh, self.hd).transpose(1, 0, 2)
            k = (hn @ l["k"].T).reshape(t, self.nkv, self.hd).transpose(1, 0, 2)
            v = (hn @ l["v"].T).reshape(t, self.nkv, self.hd).transpose(1, 0, 2)
            q, k = self.rotate(q, pos0), self.rotate(k, pos0)
            pk, pv = self.cache[li]
            k, v = np.concatenate([pk, k], 1), np.concatenate([pv, v], 1)
            self.cache[li] = (k, v)
            rep = self.nh // self.nkv
            kr, vr = np.repeat(k, rep, 0), np.repeat(v, rep, 0)         # head h uses kv head h // rep
            att = q @ kr.transpose(0, 2, 1) * self.hd ** -0.5           # [nh, t, S]
            if t != 1:
                # the prompt is processed with an empty cache: plain lower-triangular mask
                att = np.where(np.tril(np.ones((t, att.shape[2]), bool)), att, -np.inf)
            att = np.exp(att - att.max(-1, keepdims=True))
            att /= att.sum(-1, keepdims=True)
            out = (att @ vr).transpose(1, 0, 2).reshape(t, self.nh * self.hd)
            x = x + out @ l["o"].T
            hn = self.rms(x, l["rms2"])
            g, u = hn @ l["gate"].T, hn @ l["up"].T
            x = x + (g / (1.0 + np.exp(-g)) * u) @ l["down"].T
        return self.rms(x, self.norm) @ self.embed.T                    # [t, vocab]

    def generate(self, prompt, n_steps):
        ids, margins, feed, pos = [], [], list(prompt), 0
        for _ in range(n_steps + 1):
            logits = self.forward(feed, pos)[-1]
            order = np.argsort(logits)
            ids.append(int(order[-1]))
            margins.append(float(logits[order[-1]] - logits[order[-2]]))
            pos += len(feed)
            feed = [ids[-1]]
        return np.array(ids), np.array(margins)


@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("custom_softmax,fused", [(False, 0), (True, 0), (True, 1), (True, 2), (True, 3)])
def test_llama_restatement_matches_numpy_f64(cpu, cpu_ops, interleaved, custom_softmax, fused):
    """fused > 0 routes attention through the optional Ops hooks (1: causal_softmax, rope_append,
    attention_decode_flat; 2: kv_append, attention_cached; 3: also gate_up, linear_add), whose defaults (used by the CPU ops) are
    the same ops composed one by one: the graph changes shape, the values must not."""
    cfg = ug_amd.LlamaConfig(hidden_size=128, intermediate_size=320, max_position_embeddings=64, num_attention_heads=4, num_key_value_heads=2,
                             num_hidden_layers=2, vocab_size=512, rope_interleaved=interleaved)
    prompt = rng.token_ids(10, 12, cfg.vocab_size)
    want_ids, want_margins = NumpyLlama(cfg).generate(prompt.tolist(), 6)
    model = ug_amd.LlamaModel(cpu, cpu_ops, cfg, custom_softmax, seed=SEED, std=STD, fused_attention=fused)
    ids, st = model.generate(prompt, 6)
    assert ids.tolist() == want_ids.tolist()
    np.testing.assert_allclose(st["margins"], want_margins, rtol=1e-3, atol=1e-4)
    assert want_margins.min() > 1e-3   # the comparison of ids is not decided by rounding


@pytest.mark.parametrize("fused", [0, 3])
def test_llama_with_norm_vectors_around_one_matches_numpy_f64(cpu, cpu_ops, fused):
    """norm_mean = 1 (the weights of the second config-5 fixture: norm vectors 1 + N(0, std) as checkpoints hold them)."""
    cfg = ug_amd.LlamaConfig(hidden_size=128, intermediate_size=320, max_position_embeddings=64, num_attention_heads=4, num_key_value_heads=2,
                             num_hidden_layers=2, vocab_size=512)
    prompt = rng.token_ids(10, 12, cfg.vocab_size)
    want_ids, want_margins = NumpyLlama(cfg, norm_mean=1.0).generate(prompt.tolist(), 6)
    model = ug_amd.LlamaModel(cpu, cpu_ops, cfg, True, seed=SEED, std=STD, fused_attention=fused, norm_mean=1.0)
    ids, st = model.generate(prompt, 6)
    assert ids.tolist() == want_ids.tolist()
    np.testing.assert_allclose(st["margins"], want_margins, rtol=1e-3, atol=1e-4)
    plain, _ = ug_amd.LlamaModel(cpu, cpu_ops, cfg, True, seed=SEED, std=STD).generate(prompt, 6)
    assert plain.tolist() != ids.tolist()      # the option changes the model
