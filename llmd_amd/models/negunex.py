"""Negunex: a decoder-only stack of attention layers listed one by one in its configuration,
with hyper-connected residual streams.

Instead of one residual x there are S streams X_1..X_S, all equal to the embedding at the start.
Every sublayer q (1: the mixer, 2: the feed-forward) of every layer has three small learned
tensors: ``in`` [S] reads the sublayer's input u = sum_s in[s] X_s, ``mix`` [S, S] (from, to)
remixes the streams and ``out`` [S] spreads the sublayer's result over them:

    y = sublayer(layer_norm(u));   X_t <- sum_s mix[s, t] X_s + out[t] y     (all t from the old X)

The model's output is the layer norm of sum_s X_s times the head. A configuration without
``streams`` is the plain pre-norm residual, which is the case S = 1 with in = mix = out = 1.

Mixers are ``GroupedAttention`` (models/mixers.py): biased q/k/v, interleaved partial rotary with
frequency scaling, unit-RMS queries and keys, a configured score scale, value mixing with the first
value-mixing layer and a sigmoid output gate. Feed-forwards are ``GatedMLP`` (tanh-GELU) or
``ScoreMoE`` (SiLU experts, softmax scores with a selection-only correction, identity experts).

The streams, every norm and the residual arithmetic are fp32 in both activation types; ``X``
[S, T, d] is updated in place by one kernel per sublayer that also produces the next sublayer's
normed input. Attention layers cache in the runner's paged pools (one per layer).
"""
from __future__ import annotations

import torch

from llmd_amd.engine.attn_meta import AttnMeta
from llmd_amd.engine.config import ModelConfig
from llmd_amd.ops import seqmix as sm
from llmd_amd.parallel.state import get_state

from .layers import LMHead, VocabEmbedding
from .mixers import GatedMLP, GroupedAttention, ScoreMoE, _param


def make_mixer(spec: dict, d: int, eps: float, max_pos: int, device, dtype):
    t, m = spec["type"], spec["mixer"]
    if t == "attention":
        return GroupedAttention(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], m.get("rot"), eps,
                                max_pos, device, dtype, bias=True, interleaved=True, unit_norm=True,
                                v_mix=m.get("v_mix", False), gate=True)
    raise ValueError(f"unknown mixer type {t!r}")


def make_mlp(m, d: int, device, dtype):
    if m is None:
        return None
    if m["kind"] == "dense":
        return GatedMLP(d, m["ff"], "gelu_tanh", device, dtype)
    if m["kind"] == "moe":
        r = m["router"]
        return ScoreMoE(d, m["expert"]["ff"], r["experts"], r.get("identity", 0), r["top"], "silu", device, dtype)
    raise ValueError(f"unknown feed-forward kind {m['kind']!r}")


class HyperConnection(torch.nn.Module):
    """The three tensors of one sublayer's connection to the streams; fp32 copies for the kernels."""

    def __init__(self, S: int, learned: bool, device, dtype):
        super().__init__()
        self.learned = learned
        self.w_in = _param((S,), device, dtype, fill=1.0)
        self.w_out = _param((S,), device, dtype, fill=1.0)
        self.mix = torch.nn.Parameter(torch.eye(S, device=device, dtype=dtype), requires_grad=False)
        self.in32 = self.out32 = self.mix32 = None

    def finalize(self):
        self.in32, self.out32 = self.w_in.data.float(), self.w_out.data.float()
        self.mix32 = self.mix.data.float().contiguous()


class NegunexLayer(torch.nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, max_pos: int, device, dtype):
        super().__init__()
        spec = cfg.layer_specs[idx]
        d, self.eps, self.idx = cfg.hidden_size, cfg.rms_norm_eps, idx
        S, learned = max(1, cfg.hyper_streams), cfg.hyper_streams > 0
        self.mix = make_mixer(spec, d, self.eps, max_pos, device, dtype)
        self.mlp = make_mlp(spec.get("mlp"), d, device, dtype)
        self.norm1 = _param((d,), device, dtype, fill=1.0)
        self.hc1 = HyperConnection(S, learned, device, dtype)
        if self.mlp is not None:
            self.norm2 = _param((d,), device, dtype, fill=1.0)
            self.hc2 = HyperConnection(S, learned, device, dtype)


class NegunexForCausalLM(torch.nn.Module):
    supports_float32 = True
    seq_steps = True  # steps are described per sequence (AttnMeta.seq); no recurrent state

    def __init__(self, cfg: ModelConfig, device="cuda", max_pos: int = 32768, dtype=torch.bfloat16):
        super().__init__()
        if get_state().tp_size != 1:
            raise ValueError("negunex runs on one rank")
        self.cfg, self.dtype = cfg, dtype
        d = cfg.hidden_size
        self.S = max(1, cfg.hyper_streams)
        self.embed = VocabEmbedding(cfg.vocab_size, d, device, dtype=dtype)
        self.layers = torch.nn.ModuleList([NegunexLayer(cfg, i, max_pos, device, dtype)
                                           for i in range(cfg.num_hidden_layers)])
        self.norm = _param((d,), device, dtype, fill=1.0)
        self.lm_head = LMHead(cfg.vocab_size, d, device, dtype=dtype)
        self.ones = torch.ones(self.S, dtype=torch.float32, device=device)
        self.finalize()

    def finalize(self):
        """Derived constants (fp32 copies of small tensors): after every weight load."""
        for m in self.modules():
            if m is not self and hasattr(m, "finalize"):
                m.finalize()

    def attention_layers(self):
        return [l.mix for l in self.layers]

    def kv_specs(self):
        return [a.kv_spec() for a in self.attention_layers()]

    def _sublayers(self):
        """(connection, norm weight, callable) of every sublayer in order."""
        out = []
        for l in self.layers:
            out.append((l.hc1, l.norm1, l.mix, True, False))
            if l.mlp is not None:
                out.append((l.hc2, l.norm2, l.mlp, False, True))
            out[-1] = out[-1][:4] + (True,)
        return out

    @torch.no_grad()
    def forward(self, input_ids, meta: AttnMeta, layer_out=None):
        """``layer_out``: optional list that receives the sum of the streams after every layer."""
        T = input_ids.shape[0]
        d, eps, dt = self.cfg.hidden_size, self.cfg.rms_norm_eps, self.dtype
        X = torch.empty(self.S, T, d, dtype=torch.float32, device=input_ids.device)
        sm.hyper_embed(input_ids, self.embed.weight, X)
        subs = self._sublayers()
        shared = {}
        h = sm.hyper_norm(X, subs[0][0].in32, subs[0][1], eps, dt) if subs else None
        for i, (hc, _, fn, is_mixer, ends_layer) in enumerate(subs):
            y = fn(h, meta, shared) if is_mixer else fn(h)
            if i + 1 < len(subs):
                nxt_in, nxt_w = subs[i + 1][0].in32, subs[i + 1][1]
            else:
                nxt_in, nxt_w = self.ones, self.norm
            h = sm.hyper_update_norm(X, y, hc.mix32, hc.out32, nxt_in, nxt_w, eps, dt)
            if ends_layer and layer_out is not None:
                layer_out.append(X.sum(0))
        if not subs:
            h = sm.hyper_norm(X, self.ones, self.norm, eps, dt)
        return h

    @torch.no_grad()
    def compute_logits(self, h):
        # over the head's padded rows, so that the rows stay 16-byte aligned for the sampling kernel
        logits = torch.nn.functional.linear(h, self.lm_head.weight).float()
        return logits[:, :self.cfg.vocab_size]

    def weight_specs(self) -> list:
        specs = [("embed", self.embed.weight, "vocab", None), ("final.norm", self.norm, "replicate", None),
                 ("head", self.lm_head.weight, "vocab", None)]

        def add(name, p, kind="replicate", extra=None):
            specs.append((name, p, kind, extra))

        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            for q in ("1", "2"):
                if hasattr(layer, "norm" + q):
                    add(pre + "norm" + q, getattr(layer, "norm" + q))
                    hc = getattr(layer, "hc" + q)
                    if hc.learned:
                        add(f"{pre}hc{q}.in", hc.w_in)
                        add(f"{pre}hc{q}.out", hc.w_out)
                        add(f"{pre}hc{q}.mix", hc.mix)
            m, mp = layer.mix, pre + "mix."
            w, b, off = m.proj.weight, m.bias, 0
            for n, rows in (("q", m.nq), ("k", m.nk), ("v", m.nv)):
                add(mp + n, w, "fused", (off, 1, rows))
                if m.has_bias:
                    add(mp + n + ".b", b, "fused", (off, 1, rows))
                off += rows
            if m.has_gate:
                add(mp + "g", w, "fused", (off, 1, m.Hq * m.vdim))
            add(mp + "vmix", m.vmix)
            add(mp + "o", m.o.weight)
            f, fp = layer.mlp, pre + "mlp."
            if isinstance(f, GatedMLP):
                add(fp + "gate", f.gate_up.weight, "fused", (0, 1, f.ff))
                add(fp + "up", f.gate_up.weight, "fused", (f.ff, 1, f.ff))
                add(fp + "down", f.down.weight)
            elif isinstance(f, ScoreMoE):
                add(fp + "router", f.router)
                add(fp + "correction", f.correction)
                for e in range(f.E):
                    add(f"{fp}e{e}.gate", f.w1[e, :f.ff])
                    add(f"{fp}e{e}.up", f.w1[e, f.ff:])
                    add(f"{fp}e{e}.down", f.w2[e])
        return specs
