"""Mekusun: a decoder-only stack whose layers are listed one by one in its configuration.

Each layer has one mixer - latent attention, a selective scan ("mamba1") or the generalized
delta rule - and a dense (xIELU) or mixture-of-experts feed-forward or none:

    x <- x + ls1 * norm1b(mixer(norm1(x)));  x <- x + ls2 * norm2b(ff(norm2(x)))

with zero-centred RMS norms (weight 1 + w) before and after every sublayer and a per-channel
layer scale. After layer i the stream that goes on is a learned average over depth,
sum_j dwa_i[j] X_j over the embedding output X_0 and the results X_1..X_(i+1) of all layers so
far. Logits are soft-capped: c tanh(z / c).

The residual stream, the layer results X_j and all norms are fp32 in both activation types
(bfloat16 for serving, float32 for exact runs); ``hist`` [L + 2, T, d] holds X_0..X_L plus the
last average, each layer working in place in the slot its result occupies. Attention layers
cache in the paged pool, scan layers in the state pool; both are bound by the runner.
"""
from __future__ import annotations

import torch

from llmd_amd.engine.attn_meta import AttnMeta
from llmd_amd.engine.config import ModelConfig
from llmd_amd.ops import seqmix as sm
from llmd_amd.parallel.state import get_state

from .layers import LMHead, VocabEmbedding
from .mixers import ActMLP, GeneralDeltaMixer, LatentAttention, Mamba1Mixer, PlainMoE, _param


def make_mixer(spec: dict, d: int, eps: float, max_pos: int, device, dtype):
    t, m = spec["type"], spec["mixer"]
    if t == "latent_attention":
        rot = m.get("rot") or {"dims": m["rot_dim"], "base": 10000.0}
        return LatentAttention(d, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"],
                               rot["dims"], rot["base"], eps, max_pos, device, dtype)
    if t == "mamba1":
        return Mamba1Mixer(d, m["inner"], m["state"], m["dt_rank"], m["conv"], device, dtype)
    if t == "general_delta":
        if "decay_rank" not in m:
            raise ValueError("general_delta: the decay projection's rank comes from the checkpoint's tensor "
                             "shapes (ModelConfig.from_hf on the model folder) or from 'decay_rank'")
        return GeneralDeltaMixer(d, m["heads"], m["dim"], m["decay_rank"], eps, device, dtype)
    raise ValueError(f"unknown mixer type {t!r}")


def make_mlp(m, d: int, device, dtype):
    if m is None:
        return None
    if m["kind"] == "dense":
        return ActMLP(d, m["ff"], device, dtype)
    if m["kind"] == "moe":
        return PlainMoE(d, m["expert"]["ff"], m["router"]["experts"], m["router"]["top"], device, dtype)
    raise ValueError(f"unknown feed-forward kind {m['kind']!r}")


class MekusunLayer(torch.nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, max_pos: int, device, dtype):
        super().__init__()
        spec = cfg.layer_specs[idx]
        d, self.eps, self.idx = cfg.hidden_size, cfg.rms_norm_eps, idx
        self.mix = make_mixer(spec, d, self.eps, max_pos, device, dtype)
        self.mlp = make_mlp(spec.get("mlp"), d, device, dtype)
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if self.mlp is not None else ()):
            setattr(self, n, _param((d,), device, dtype, fill=0.0))
        self.ls1 = _param((d,), device, dtype, fill=1.0)
        if self.mlp is not None:
            self.ls2 = _param((d,), device, dtype, fill=1.0)
        dwa = torch.zeros(idx + 2, device=device, dtype=dtype)
        dwa[-1] = 1.0
        self.dwa = torch.nn.Parameter(dwa, requires_grad=False)
        self.dwa32 = None

    def finalize(self):
        self.dwa32 = self.dwa.data.float()

    def forward(self, h, x, meta: AttnMeta, dt):
        """h = norm1(x) (from the previous pass over x); x is updated in place to the layer's result."""
        y = self.mix(h, meta)
        if self.mlp is None:
            sm.add_post_norm(y, self.norm1b, self.ls1, x, self.eps)
            return
        h = sm.add_post_norm(y, self.norm1b, self.ls1, x, self.eps, self.norm2, dt)
        sm.add_post_norm(self.mlp(h), self.norm2b, self.ls2, x, self.eps)


class MekusunForCausalLM(torch.nn.Module):
    supports_float32 = True
    stateful = True  # scan layers: no prefix reuse, one state slot per running sequence

    def __init__(self, cfg: ModelConfig, device="cuda", max_pos: int = 32768, dtype=torch.bfloat16):
        super().__init__()
        if get_state().tp_size != 1:
            raise ValueError("mekusun runs on one rank (its scan layers are not tensor-parallel)")
        self.cfg, self.dtype = cfg, dtype
        d = cfg.hidden_size
        self.embed = VocabEmbedding(cfg.vocab_size, d, device, dtype=dtype)
        self.layers = torch.nn.ModuleList([MekusunLayer(cfg, i, max_pos, device, dtype)
                                           for i in range(cfg.num_hidden_layers)])
        self.norm = _param((d,), device, dtype, fill=0.0)
        self.lm_head = LMHead(cfg.vocab_size, d, device, dtype=dtype)
        self.finalize()

    def finalize(self):
        """Derived constants (fp32 copies, -exp(A_log), activation numbers): after every weight load."""
        for m in self.modules():
            if m is not self and hasattr(m, "finalize"):
                m.finalize()

    def attention_layers(self):
        return [l.mix for l in self.layers if isinstance(l.mix, LatentAttention)]

    def state_layers(self):
        return [l.mix for l in self.layers if hasattr(l.mix, "state_shapes")]

    def kv_specs(self):
        return [a.kv_spec() for a in self.attention_layers()]

    @torch.no_grad()
    def forward(self, input_ids, meta: AttnMeta, layer_out=None):
        """``layer_out``: optional list that receives a copy of the stream after every layer
        (after the depth average), for layer-by-layer checks."""
        T, L = input_ids.shape[0], len(self.layers)
        d, eps, dt = self.cfg.hidden_size, self.cfg.rms_norm_eps, self.dtype
        hist = torch.empty(L + 2, T, d, dtype=torch.float32, device=input_ids.device)
        sm.embed_scale(input_ids, self.embed.weight, self.cfg.embedding_scale, hist)
        h = sm.zc_norm(hist[1], self.layers[0].norm1, eps, dt)
        for i, layer in enumerate(self.layers):
            layer(h, hist[i + 1], meta, dt)
            nxt = self.layers[i + 1].norm1 if i + 1 < L else self.norm
            h = sm.depth_avg_norm(hist, i + 2, layer.dwa32, i + 2, nxt, eps, dt)
            if layer_out is not None:
                layer_out.append(hist[i + 2].clone())
        return h

    @torch.no_grad()
    def compute_logits(self, h):
        # over the head's padded rows, so that the rows stay 16-byte aligned for the sampling kernel
        logits = torch.nn.functional.linear(h, self.lm_head.weight).float()
        if self.cfg.logit_softcap:
            sm.softcap_(logits, self.cfg.logit_softcap)
        return logits[:, :self.cfg.vocab_size]

    def weight_specs(self) -> list:
        specs = [("embed", self.embed.weight, "vocab", None), ("final.norm", self.norm, "replicate", None),
                 ("head", self.lm_head.weight, "vocab", None)]

        def add(name, p, kind="replicate", extra=None):
            specs.append((name, p, kind, extra))

        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            for n in ("norm1", "norm1b", "norm2", "norm2b", "ls1", "ls2", "dwa"):
                if hasattr(layer, n):
                    add(pre + n, getattr(layer, n))
            m, mp = layer.mix, pre + "mix."
            if isinstance(m, LatentAttention):
                for n, p in (("q", m.q.weight), ("dkv", m.dkv.weight), ("dkv.norm", m.dkv_norm), ("uk", m.uk),
                             ("uv", m.uv), ("o", m.o.weight)):
                    add(mp + n, p)
            elif isinstance(m, Mamba1Mixer):
                for n, p in (("in", m.in_proj.weight), ("conv", m.conv), ("conv.b", m.conv_b), ("x", m.x_proj.weight),
                             ("dt", m.dt_proj.weight), ("dt.b", m.dt_b), ("A_log", m.A_log), ("D", m.D),
                             ("o", m.o.weight)):
                    add(mp + n, p)
            else:
                HD = m.H * m.d
                for j, n in enumerate(("r", "k", "v", "g", "a")):
                    add(mp + n, m.proj.weight, "fused", (j * HD, 1, HD))
                add(mp + "w1", m.proj.weight, "fused", (5 * HD, 1, m.wr))
                for n, p in (("a.b", m.a_b), ("w2", m.w2.weight), ("w0", m.w0), ("norm", m.norm), ("o", m.o.weight)):
                    add(mp + n, p)
            f, fp = layer.mlp, pre + "mlp."
            if isinstance(f, ActMLP):
                for n, p in (("up", f.up.weight), ("down", f.down.weight), ("act", f.act)):
                    add(fp + n, p)
            elif isinstance(f, PlainMoE):
                add(fp + "router", f.router)
                add(fp + "router.b", f.router_b)
                for e in range(f.E):
                    add(f"{fp}e{e}.up", f.w1[e])
                    add(f"{fp}e{e}.down", f.w2[e])
        return specs
