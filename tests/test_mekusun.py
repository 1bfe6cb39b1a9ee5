"""Mekusun on the engine against the plain float64 oracle (tests/mekusun_oracle.py): every mixer and
feed-forward alone, whole prompts against token-by-token decoding and portions down to two tokens,
mixed batches of unequal requests with pages and state slots that are freed and reused, page
borders, the first token, long decoding, odd sizes, greedy generation through the scheduler.
Each case runs on the CPU reference ops and, marked gpu, on the HIP kernels."""
import json
import math
import os

import pytest
import torch
from safetensors.torch import save_file

import mekusun_oracle as oracle
from llmd_amd.engine.config import EngineConfig, ModelConfig
from llmd_amd.engine.engine import LLMEngine
from llmd_amd.engine.request import SamplingParams

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def attn(heads, dim, rot_dim, vdim, rank, rot_dims=None, base=10000.0):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
                      "scale": 1.0 / math.sqrt(dim + rot_dim), "rot": {"dims": rot_dims or rot_dim, "base": base}}}


def mamba(inner, state, dt_rank, conv):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}}


def delta(heads, dim):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(layers, width=48, vocab=70, scale=3.0, cap=20.0, eps=1e-5):
    return {"architecture": "Mekusun", "width": width, "vocab": vocab, "embedding": {"scale": scale},
            "logit_softcap": cap, "norm": {"eps": eps},
            "layers": [dict(l, mlp=f) for l, f in layers]}


# sizes that differ from each other wherever the design lets them: unrotated != rotated != value
# != latent size, rotary over a part of the rotated dims, two attention layers of different
# geometry, a state size that is no power of two, a delta head that is no multiple of 32
MIXED = config([(attn(3, 24, 8, 16, 40, rot_dims=4, base=500.0), dense(72)),
                (delta(3, 20), moe(24, 5, 2)),
                (mamba(56, 6, 5, 4), moe(40, 3, 1)),
                (attn(5, 8, 12, 20, 24), None),
                (mamba(40, 70, 3, 2), dense(36))], width=48, vocab=70)
# values the first configuration keeps apart, made equal or 1 here
PLAIN = config([(mamba(32, 1, 1, 1), None),
                (attn(1, 16, 16, 16, 16), moe(16, 4, 4)),
                (delta(1, 64), dense(64))], width=32, vocab=64, scale=1.0, cap=0.0)
# sizes that are multiples of nothing: vector loads, MFMA padding and lane groups all take their slow paths
ODD = config([(attn(7, 10, 6, 14, 18, base=77.0), moe(22, 7, 3)),
              (delta(2, 50), dense(26)),
              (mamba(30, 3, 2, 5), None),
              (mamba(20, 100, 7, 2), moe(10, 2, 2))], width=34, vocab=51, scale=0.5, cap=7.0, eps=1e-4)
NO_ATTENTION = config([(delta(2, 16), dense(40)), (mamba(24, 8, 4, 3), None)], width=24, vocab=40)


def model_dir(tmp_path, cfg, seed=0, decay_rank=6):
    W = oracle.random_weights(cfg, seed, decay_rank)
    d = tmp_path / f"m{seed}"
    d.mkdir(exist_ok=True)
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    return str(d), W


def engine(path, device, dtype="float32", pages=16, seqs=4, **kw):
    mc = ModelConfig.from_hf(path)
    cfg = EngineConfig.create(path, model_config=mc, device=device, dtype=dtype, load_format="safetensors",
                              weights_path=path, block_size=64, num_gpu_blocks=pages, max_num_seqs=seqs,
                              max_model_len=pages * 64 + 1, max_num_batched_tokens=pages * 64,
                              enforce_eager=True, prefill_token_align=0, **kw)
    return LLMEngine(cfg, capture_graphs=False)


def rel_err(got, want):
    d = got.double().cpu() - want
    return float(torch.sqrt((d * d).mean(-1)).max() / torch.sqrt((want * want).mean()))


def replay(eng, prompts, steps):
    """steps: list of lists of (name, count). Returns name -> logits [len, vocab] (all positions)."""
    at = {n: 0 for n in prompts}
    out = {n: [] for n in prompts}
    for step in steps:
        entries, end = [], []
        for n, c in step:
            toks = prompts[n][at[n]:at[n] + c]
            entries.append((n, toks, list(range(len(toks)))))
            at[n] += c
            if at[n] == len(prompts[n]):
                end.append(n)
        lg = eng.forced_step(entries, end)
        o = 0
        for n, c in step:
            out[n].append(lg[o:o + c].cpu())
            o += c
    return {n: torch.cat(v) for n, v in out.items() if v}


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


TOL = {"float32": 2e-4, "bfloat16": 6e-2}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layer", [(attn(3, 24, 8, 16, 40, rot_dims=4), dense(72)), (mamba(56, 6, 5, 4), moe(24, 5, 2)),
                                   (delta(3, 20), None), (mamba(40, 70, 3, 1), dense(20)), (delta(2, 40), moe(8, 3, 3))],
                         ids=["latent+dense", "mamba+moe", "delta", "mamba-wide-state+dense", "delta+moe"])
def test_each_mechanism_alone(tmp_path, device, layer):
    cfg = config([layer])
    path, W = model_dir(tmp_path, cfg)
    toks = tokens(70, cfg["vocab"], 1)
    want = oracle.forward(cfg, W, toks)
    got = replay(engine(path, device), {"a": toks}, [[("a", 70)]])["a"]
    assert rel_err(got, want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_layer_streams(tmp_path, device):
    """The stream after every layer (after the depth average), not only the logits."""
    from llmd_amd.engine.attn_meta import AttnMeta

    path, W = model_dir(tmp_path, MIXED)
    toks = tokens(40, MIXED["vocab"], 2)
    streams = []
    oracle.forward(MIXED, W, toks, streams)
    eng = engine(path, device)
    r = eng.runner
    pl = {"graph": False, "nd": 0, "ids": toks, "pos": list(range(40)), "slots": list(range(40)),
          "d_bt": __import__("numpy").zeros((0, r.width), "int32"), "d_len": __import__("numpy").zeros(0, "int32"),
          "p_ql": [40], "p_ctx": [40], "p_bt": __import__("numpy").zeros((1, r.width), "int32"), "rows": [],
          "seq": ([0], [0])}
    ids, meta = r._eager_meta(pl)
    assert isinstance(meta, AttnMeta) and meta.seq.num_seqs == 1
    got = []
    r.model(ids, meta, layer_out=got)
    for i, (g, w) in enumerate(zip(got, streams)):
        assert rel_err(g, w) < 1e-4, i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_decode_and_portions_agree(tmp_path, device, dtype):
    path, W = model_dir(tmp_path, MIXED)
    toks = tokens(150, MIXED["vocab"], 3)
    want = oracle.forward(MIXED, W, toks)
    tol = TOL[dtype]
    whole = replay(engine(path, device, dtype), {"a": toks}, [[("a", 150)]])["a"]
    assert rel_err(whole, want) < tol
    # a short prompt, then 140 tokens one by one over two page borders
    dec = replay(engine(path, device, dtype), {"a": toks}, [[("a", 10)]] + [[("a", 1)]] * 140)["a"]
    assert rel_err(dec, want) < tol
    # portions that end just before, at and just after the page borders, down to two and one tokens
    cuts = [2, 61, 1, 3, 2, 58, 1, 1, 2, 19]
    assert sum(cuts) == 150
    por = replay(engine(path, device, dtype), {"a": toks}, [[("a", c)] for c in cuts])["a"]
    assert rel_err(por, want) < tol
    if dtype == "float32":  # the three ways differ by rounding only
        assert rel_err(dec, whole.double()) < 1e-4 and rel_err(por, whole.double()) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_reuse_pages_and_slots(tmp_path, device):
    """Five unequal requests through three state slots and seven pages: portions beside single
    tokens, requests that pause, end and hand their pages and slot to the next one."""
    path, W = model_dir(tmp_path, MIXED)
    lens = {"a": 130, "b": 1, "c": 67, "d": 90, "e": 64}
    prompts = {n: tokens(k, MIXED["vocab"], 10 + i) for i, (n, k) in enumerate(lens.items())}
    steps = [[("a", 60), ("b", 1), ("c", 2)],
             [("c", 1), ("a", 4)],
             [("a", 1), ("c", 62), ("d", 30)],           # b's slot and page reused by d
             [("d", 1), ("a", 63)],                      # a reaches 128: exactly two pages
             [("c", 1), ("d", 34), ("a", 1)],
             [("c", 1), ("a", 1), ("d", 25)],            # all three end: every page and slot is free again
             [("e", 3)],
             [("e", 61)],
             ]
    eng = engine(path, device, pages=7, seqs=3)
    got = replay(eng, prompts, steps)
    for n in prompts:
        assert got[n].shape[0] == lens[n], n
        assert rel_err(got[n], oracle.forward(MIXED, W, prompts[n])) < TOL["float32"], n
    eng.bm.check_invariants()
    assert eng.bm.num_free() == 7 and eng.bm.slots.num_free() == 3
    # each alone gives the same rows up to rounding
    alone = replay(engine(path, device, pages=6, seqs=3), {"d": prompts["d"]}, [[("d", 90)]])["d"]
    assert rel_err(got["d"], alone.double()) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cfg", [PLAIN, NO_ATTENTION, ODD], ids=["equal-or-one", "no-attention", "odd"])
def test_other_sizes(tmp_path, device, cfg, dtype):
    path, W = model_dir(tmp_path, cfg, seed=5)
    toks = tokens(80, cfg["vocab"], 6)
    want = oracle.forward(cfg, W, toks)
    got = replay(engine(path, device, dtype), {"a": toks},
                 [[("a", 5)], [("a", 60)], [("a", 2)]] + [[("a", 1)]] * 13)["a"]
    assert rel_err(got, want) < TOL[dtype]


def _paged(keys, block_size, device, dtype):
    """Scatter key rows over shuffled pages; returns (cache, table)."""
    n, dk = keys.shape
    nb = -(-n // block_size)
    perm = torch.randperm(nb + 3, generator=torch.Generator().manual_seed(1))[:nb]
    cache = torch.randn(nb + 3, block_size, dk, generator=torch.Generator().manual_seed(2)).to(dtype)
    for i in range(n):
        cache[perm[i // block_size], i % block_size] = keys[i].to(dtype)
    return cache.to(device), perm.int().view(1, -1).to(device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("where", ["far", "page-end", "page-start", "last-seen", "first-unseen"])
def test_one_key_stands_out(device, where):
    """One key among 300 has a score far above the rest: the output is its latent if and only
    if the row may see it - far back, on either side of a page border, the last visible key, and
    the first one beyond the row's length."""
    from llmd_amd.ops import seqmix as sm

    R, dr, H, n, seen = 24, 8, 3, 300, 200
    g = torch.Generator().manual_seed(7)
    keys = torch.randn(n, R + dr, generator=g) * 0.3
    q = torch.randn(1, H, R + dr, generator=g) * 0.3
    j = {"far": 2, "page-end": 63, "page-start": 64, "last-seen": seen - 1, "first-unseen": seen}[where]
    keys[j] = q[0, 1] / q[0, 1].norm() * 12.0          # head 1 looks straight at key j
    q[0, 1] *= 6.0
    cache, table = _paged(keys, 64, device, torch.float32)
    out = sm.latent_attention(q.to(device), cache, table, torch.zeros(1, dtype=torch.int32, device=device),
                              torch.tensor([seen], dtype=torch.int32, device=device), 1.0, R)
    s = torch.einsum("hd,nd->hn", q[0].double(), keys[:seen].double())
    want = torch.softmax(s, -1) @ keys[:seen, :R].double()
    assert rel_err(out[0], want) < 1e-4
    hit = torch.allclose(out[0, 1].cpu().double(), keys[j, :R].double(), atol=1e-2)
    assert hit == (where != "first-unseen")


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    path, W = model_dir(tmp_path, MIXED, seed=8)
    prompts = [tokens(9, MIXED["vocab"], 20), tokens(70, MIXED["vocab"], 21), tokens(1, MIXED["vocab"], 22)]
    eng = engine(path, device, pages=8, seqs=2, async_scheduling=False)  # 3 requests over 2 slots
    reqs = eng.generate(prompts, SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    for p, r in zip(prompts, reqs):
        seq = list(p)
        for _ in range(6):
            seq.append(int(oracle.forward(MIXED, W, seq)[-1].argmax()))
        assert r.output_token_ids == seq[len(p):]
    eng.bm.check_invariants()
    assert eng.bm.slots.num_free() == 2


@pytest.mark.gpu
@pytest.mark.parametrize("E,k", [(5, 2), (64, 6), (130, 8), (16, 16), (600, 3)])
def test_router_top_k(E, k):
    from llmd_amd.ops import seqmix as sm

    g = torch.Generator().manual_seed(E)
    z = torch.randn(37, E, generator=g)
    z[3, 1] = z[3, 0] = z[3].max() + 1.0          # a tie: the lower index comes first
    ids, w = sm.moe_route(z.cuda(), k)
    order = sorted(range(E), key=lambda e: (-float(z[3, e]), e))[:k]
    assert ids[3].tolist() == order
    top, idx = z.topk(k, -1)
    assert torch.equal(ids.cpu().long().sort(-1).values, idx.sort(-1).values)
    assert torch.allclose(w.cpu().sum(-1), torch.ones(37), atol=1e-6)
    assert torch.allclose(w.cpu().sort(-1, descending=True).values, torch.softmax(top, -1), atol=1e-6)


def test_state_slots_and_block_manager():
    from llmd_amd import _rt_loader
    from llmd_amd.engine.state_cache import StatefulBlockManager

    bm = StatefulBlockManager(_rt_loader.rt().BlockManager(4, 64, False, False), 2)
    import numpy as np

    t = np.zeros(10, dtype=np.int32)
    for s in (1, 2, 3):
        assert bm.acquire(s, t, 0) == 0
    assert bm.grow(1, 65) and bm.grow(2, 10)
    assert bm.state_slot(1) != bm.state_slot(2)
    assert not bm.grow(3, 10)                       # no slot left; nothing taken
    assert bm.num_free() == 1
    assert not bm.grow(2, 64 * 3)                   # pages short; the slot stays
    first = bm.state_slot(1)
    bm.free(1)
    assert bm.grow(3, 100) and bm.state_slot(3) == first
    bm.free(2), bm.free(3)
    bm.check_invariants()
    assert bm.num_free() == 4 and bm.slots.num_free() == 2


def test_config_reads_sizes_from_file_and_shapes(tmp_path):
    path, _ = model_dir(tmp_path, MIXED, decay_rank=11)
    mc = ModelConfig.from_hf(path)
    assert mc.model_type == "mekusun" and mc.hidden_size == 48 and mc.vocab_size == 70
    assert mc.layer_specs[1]["mixer"]["decay_rank"] == 11
    assert mc.embedding_scale == 3.0 and mc.logit_softcap == 20.0
    assert os.path.exists(os.path.join(path, "model.safetensors"))


@pytest.mark.gpu
@pytest.mark.parametrize("decode_only", [False, True], ids=["mixed-step", "decode-step"])
@pytest.mark.parametrize("H,R,dr", [(3, 40, 8), (5, 24, 12), (6, 64, 16), (16, 512, 64), (2, 100, 30)])
def test_matrix_core_attention_matches_fp32(H, R, dr, decode_only):
    """bfloat16 attention on the matrix cores against the fp32 kernel on the same (bf16-rounded)
    inputs: a prompt portion that continues a context, a whole prompt and two decode rows in one
    step, over shuffled pages; sizes that need padding to the MFMA shapes included."""
    from llmd_amd.engine.attn_meta import SeqMeta
    from llmd_amd.ops import seqmix as sm

    dev, bs, Dk = "cuda", 64, R + dr
    g = torch.Generator().manual_seed(H * 1000 + R)
    # (context before the run, run length): decodes first, then the portions
    runs = [(130, 1), (63, 1), (70, 37), (0, 90)]
    if decode_only:  # long contexts, one token each: the keys are cut into ranges and merged
        runs = [(700, 1), (300, 1), (63, 1), (1500, 1), (0, 1)]
    nblk = [-(-(c + n) // bs) for c, n in runs]
    perm = torch.randperm(sum(nblk) + 2, generator=g)
    tables = torch.zeros(len(runs), max(nblk), dtype=torch.int32)
    o = 0
    for i, k in enumerate(nblk):
        tables[i, :k] = perm[o:o + k]
        o += k
    cache = (torch.randn(sum(nblk) + 2, bs, Dk, generator=g) * 0.5).to(torch.bfloat16)
    T = sum(n for _, n in runs)
    q = (torch.randn(T, H, Dk, generator=g) * 0.7).to(torch.bfloat16)
    row_seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, (_, n) in enumerate(runs)])
    row_len = torch.cat([torch.arange(c + 1, c + n + 1, dtype=torch.int32) for c, n in runs])
    start = torch.tensor([0] + list(torch.tensor([n for _, n in runs]).cumsum(0)), dtype=torch.int32)
    nz = torch.zeros(len(runs), dtype=torch.int32, device=dev)
    seq = SeqMeta(num_seqs=len(runs), seq_start=start.to(dev), seq_slot=nz, seq_init=nz, row_seq=row_seq.to(dev),
                  row_len=row_len.to(dev), tables=tables.to(dev), max_len=int(row_len.max()),
                  max_q=max(n for _, n in runs), q_lens=[n for _, n in runs])
    scale = Dk ** -0.5
    fast = sm.latent_attention(q.to(dev), cache.to(dev), seq.tables, seq.row_seq, seq.row_len, scale, R, 4, seq=seq)
    slow = sm.latent_attention(q.float().to(dev), cache.float().to(dev), seq.tables, seq.row_seq, seq.row_len, scale, R, 4)
    assert fast.dtype == torch.bfloat16
    err = (fast.float() - slow).abs().max() / slow.abs().max()
    assert float(err) < 8e-3, float(err)


@pytest.mark.gpu
@pytest.mark.parametrize("T,d,F,E,k", [(70, 48, 24, 5, 2), (300, 256, 200, 16, 3), (9, 64, 72, 4, 4), (33, 50, 30, 3, 1),
                                       (1500, 256, 328, 4, 2)])  # the last: prompt-sized, the wide tiles
def test_expert_gemm_bf16_matches_fp32(T, d, F, E, k):
    """The bfloat16 expert feed-forward (matrix cores where rows are 16-byte aligned, the FMA
    kernel otherwise) against the float32 kernels on the same bf16-rounded inputs."""
    from llmd_amd.ops import seqmix as sm

    g = torch.Generator().manual_seed(T + d)
    h = torch.randn(T, d, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(E, F, d, generator=g) / math.sqrt(d)).to(torch.bfloat16)
    w2 = (torch.randn(E, d, F, generator=g) / math.sqrt(F)).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g).cuda()
    ids, w = sm.moe_route(logits, k)
    top, idx = logits.topk(k, -1)
    assert torch.equal(ids.long(), idx) and torch.allclose(w, torch.softmax(top, -1), atol=1e-6)
    fast = sm.moe_ffn(h.cuda(), ids, w, w1.cuda(), w2.cuda())
    slow = sm.moe_ffn(h.float().cuda(), ids, w, w1.float().cuda(), w2.float().cuda())
    want = torch.zeros(T, d, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            want[t] += float(w[t, j]) * (oracle.gelu_erf(h[t].double() @ w1[e].double().T) @ w2[e].double().T)
    assert float((slow.cpu().double() - want).abs().max() / want.abs().max()) < 1e-5
    assert float((fast.float() - slow).abs().max() / slow.abs().max()) < 2e-2


def test_trace_runner_program(tmp_path):
    """bin/trace_run as a program: steps on standard input, 'done <step>' lines, one fp32 file per step
    with wanted places; a request that skips a step, ends, and a later one that reuses its slot."""
    import subprocess
    import sys

    import numpy as np

    path, W = model_dir(tmp_path, NO_ATTENTION, seed=3)
    a, b, c = (tokens(n, NO_ATTENTION["vocab"], 40 + i) for i, n in enumerate((9, 3, 5)))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}, {"id": "b", "tokens": b[:2], "want": []}],
              "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[6:7], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[2:], "want": [0]}, {"id": "a", "tokens": a[7:], "want": [1]}],
              "end": ["a", "b"]},
             {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [4]}], "end": ["c"]}]
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128", "--max-seqs", "2", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    V = NO_ATTENTION["vocab"]
    la, lb, lc = (oracle.forward(NO_ATTENTION, W, t) for t in (a, b, c))
    want = {0: torch.stack([la[0], la[5]]), 1: la[6:7], 2: torch.stack([lb[2], la[8]]), 3: lc[4:5]}
    for i, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V).copy())
        assert got.shape == w.shape and rel_err(got, w) < TOL["float32"], i


@pytest.mark.parametrize("async_sched", [False, True], ids=["sync", "async"])
def test_preemption_recomputes_state(tmp_path, async_sched):
    """A pool too small for both requests' growth: one is preempted (pages and state slot freed),
    recomputed from its first token, and still generates what an unconstrained engine generates."""
    path, _ = model_dir(tmp_path, MIXED, seed=9)
    prompts = [tokens(50, MIXED["vocab"], 30), tokens(50, MIXED["vocab"], 31)]
    sp = SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)
    roomy = engine(path, "cpu", pages=8, seqs=2, async_scheduling=async_sched)
    want = [r.output_token_ids for r in roomy.generate(prompts, sp)]
    tight = engine(path, "cpu", pages=2, seqs=2, async_scheduling=async_sched)
    got = [r.output_token_ids for r in tight.generate(prompts, sp)]
    assert tight.sched.num_preemptions_total > 0
    assert got == want
    tight.bm.check_invariants()
    assert tight.bm.num_free() == 2 and tight.bm.slots.num_free() == 2
