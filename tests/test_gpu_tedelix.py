"""Tedelix on the GPU against the plain implementation (``plain_tedelix.py``): every mechanism
alone, then whole models of two small configurations that differ in every size, through every
way of cutting requests into steps, through pages and state slots that are used again, and
through ``LLM.generate``.  Weights are drawn here with deviations that make activations of order
one (sharp softmaxes, states that matter), and a few tests build inputs so that one key decides."""
import json
import math
import os

import numpy as np
import pytest
import torch

import plain_tedelix as P
from helpers import cut_mixed, cut_portions, cut_tail_single, cut_whole, random_requests, run_steps

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

CONFIGS = {
    # small heads, grouped queries, a window of one position, a layer without feed-forward
    "P": dict(architecture="Tedelix", vocab=200, width=64, norm=dict(eps=1e-5), logit_scale=0.7, logit_softcap=12.0, layers=[
        dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=16, vdim=24, mask=dict(size=9), scale=0.3,
                                          rot=dict(base=1000.0, dims=8)), mlp=dict(kind="dense", ff=96)),
        dict(type="lightning", mixer=dict(heads=2, dim=16, vdim=8, decay=[0.9, 0.5]), mlp=None),
        dict(type="general_delta", mixer=dict(heads=2, dim=16), mlp=dict(kind="dense", ff=40)),
        dict(type="attention", mixer=dict(heads=3, kv_heads=3, dim=20, vdim=36, mask=dict(size=1), scale=1.0,
                                          rot=dict(base=77.0, dims=20)), mlp=dict(kind="dense", ff=24)),
        dict(type="lightning", mixer=dict(heads=1, dim=36, vdim=70, decay=[0.97]), mlp=dict(kind="dense", ff=8)),
    ]),
    # heads beyond one 64-wide slice, key rows beyond one thread's 32, state layers first and last
    "Q": dict(architecture="Tedelix", vocab=333, width=136, norm=dict(eps=1e-6), logit_scale=1.3, logit_softcap=50.0, layers=[
        dict(type="general_delta", mixer=dict(heads=3, dim=72), mlp=dict(kind="dense", ff=200)),
        dict(type="attention", mixer=dict(heads=8, kv_heads=2, dim=72, vdim=132, mask=dict(size=40), scale=0.11,
                                          rot=dict(base=50000.0, dims=72)), mlp=None),
        dict(type="lightning", mixer=dict(heads=3, dim=40, vdim=72, decay=[0.999, 0.8, 0.3]), mlp=dict(kind="dense", ff=64)),
        dict(type="attention", mixer=dict(heads=2, kv_heads=1, dim=32, vdim=16, mask=dict(size=200), scale=0.25,
                                          rot=dict(base=10000.0, dims=4)), mlp=dict(kind="dense", ff=136)),
        dict(type="general_delta", mixer=dict(heads=1, dim=128), mlp=None),
    ]),
    # a width and a vocabulary that are no multiples of eight, three and six query heads a key/value head
    "R": dict(architecture="Tedelix", vocab=211, width=100, norm=dict(eps=1e-6), logit_scale=1.0, logit_softcap=8.0, layers=[
        dict(type="attention", mixer=dict(heads=3, kv_heads=1, dim=24, vdim=40, mask=dict(size=21), scale=0.2,
                                          rot=dict(base=500.0, dims=12)), mlp=dict(kind="dense", ff=50)),
        dict(type="general_delta", mixer=dict(heads=5, dim=20), mlp=dict(kind="dense", ff=30)),
        dict(type="attention", mixer=dict(heads=12, kv_heads=2, dim=16, vdim=18, mask=dict(size=64), scale=0.25,
                                          rot=dict(base=10000.0, dims=16)), mlp=None),
        dict(type="lightning", mixer=dict(heads=5, dim=20, vdim=12, decay=[0.9, 0.8, 0.7, 0.6, 0.5]), mlp=dict(kind="dense", ff=77)),
    ]),
}
DECAY_RANK = {"P": 4, "Q": 12, "R": 7}
PAGE = {"P": 8, "Q": 16, "R": 16}


def bf16_round(a: np.ndarray) -> torch.Tensor:
    return torch.tensor(a, dtype=torch.float32).to(torch.bfloat16)


def draw_weights(cfg: dict, rank: int, seed: int):
    """name -> bfloat16 tensor for every tensor of the design, activations of order one."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    mat = lambda o, i: bf16_round(rng.standard_normal((o, i)) / math.sqrt(i))
    vec = lambda n, mean, std: bf16_round(mean + std * rng.standard_normal(n))
    t = {"embed": bf16_round(rng.standard_normal((cfg["vocab"], W))), "final.norm": vec(W, 1.0, 0.1)}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        t[p + "norm1"] = vec(W, 1.0, 0.1)
        if layer["type"] == "attention":
            t[p + "mix.q"], t[p + "mix.k"] = mat(m["heads"] * m["dim"], W), mat(m["kv_heads"] * m["dim"], W)
            t[p + "mix.v"], t[p + "mix.o"] = mat(m["kv_heads"] * m["vdim"], W), mat(W, m["heads"] * m["vdim"])
        elif layer["type"] == "lightning":
            hk, hv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"], t[p + "mix.g"] = mat(hk, W), mat(hk, W), mat(hv, W), mat(hv, W)
            t[p + "mix.o"], t[p + "mix.norm"] = mat(W, hv), vec(hv, 1.0, 0.1)
        else:
            hd = m["heads"] * m["dim"]
            for n in "rkvga":
                t[p + "mix." + n] = mat(hd, W)
            t[p + "mix.a.b"], t[p + "mix.w0"] = vec(hd, 0.0, 1.0), vec(hd, 0.0, 1.5)
            t[p + "mix.w1"], t[p + "mix.w2"] = mat(rank, W), mat(hd, rank)
            t[p + "mix.norm"], t[p + "mix.o"] = vec(hd, 1.0, 0.1), mat(W, hd)
        if layer["mlp"] is not None:
            t[p + "mlp.up"], t[p + "mlp.down"] = mat(layer["mlp"]["ff"], W), mat(W, layer["mlp"]["ff"])
    return t


@pytest.fixture(scope="module")
def tdirs(tmp_path_factory):
    from rustinfer_amd.weights import write_safetensors
    out = {}
    for k, (name, cfg) in enumerate(CONFIGS.items()):
        d = str(tmp_path_factory.mktemp("tedelix_" + name))
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(cfg, f)
        write_safetensors(os.path.join(d, "model.safetensors"), draw_weights(cfg, DECAY_RANK[name], 11 + k))
        out[name] = d
    return out


@pytest.fixture(scope="module")
def plain(tdirs):
    return {name: P.read_model(d) for name, d in tdirs.items()}


@pytest.fixture(scope="module")
def plain_logits(plain):
    """(name, request lengths, seed) -> {request: logits of the whole request}, computed once."""
    memo = {}

    def get(name, lengths, seed):
        key = (name, tuple(lengths), seed)
        if key not in memo:
            cfg, w = plain[name]
            reqs = random_requests(cfg["vocab"], lengths, seed)
            memo[key] = (reqs, {rid: P.forward(cfg, w, toks) for rid, toks in reqs.items()})
        return memo[key]
    return get


def engine_for(model_dir, dtype, name, num_pages=64, max_requests=4, max_len=512):
    from rustinfer_amd.engine import build_engine
    return build_engine(model_dir, dtype=dtype, device=DEV, page_size=PAGE[name], num_pages=num_pages,
                        max_requests=max_requests, max_model_len=max_len, max_batch_tokens=2048)


# a row of logits: root mean square of the difference (its mean taken off) over the deviation of
# the plain logits.  32-bit rounds at 1e-7; bfloat16 at 4e-3 per rounding, and a wrong key, a window
# one position off or a lost state gives 0.1 and more with these weights.
TOL = {"float32": 2e-4, "bfloat16": 6e-2}


def check_rows(steps, results, logits, dtype, label):
    s = max(float(np.std(v)) for v in logits.values())
    pos, worst = {}, 0.0
    for st in steps:
        got, row = results.get(st["step"]), 0
        for e in st["entries"]:
            p0 = pos.get(e["id"], 0)
            for w in e["want"]:
                d = got[row].astype(np.float64) - logits[e["id"]][p0 + w]
                err = float(np.sqrt(np.mean((d - d.mean()) ** 2))) / s
                assert err <= TOL[dtype], (f"{label}: step {st['step']} request {e['id']} position {p0 + w} (place {w} of a "
                                           f"portion of {len(e['tokens'])} from {p0}): row error {err:.2e} of the deviation")
                worst, row = max(worst, err), row + 1
            pos[e["id"]] = p0 + len(e["tokens"])
        for rid in st["end"]:
            pos.pop(rid, None)
    return worst


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
class OnePart:
    """The least a 'model' must be for the engine to build a step context around one mixer."""
    vocab_size = 100

    def __init__(self, mixer, pos_encs=()):
        self.mixer, self.pos_encs = mixer, list(pos_encs)

    def prepare(self, rt, max_positions):
        for pe in self.pos_encs:
            pe.prepare(rt, max_positions)

    def cache_needs(self):
        need = self.mixer.cache_need()
        return {0: need} if need is not None else {}


def run_part(part, pos_encs, dtype, x, cuts, page=8, batch_with=None):
    """The part's output [T, hidden] for one sequence ``x [T, hidden]`` fed in portions of ``cuts``.
    ``batch_with``: rows of a second request that shares every step (its output is dropped)."""
    from rustinfer_amd.engine import Engine, StepEntry, make_runtime
    rt = make_runtime(dtype, DEV)
    eng = Engine(OnePart(part, pos_encs), rt, page_size=page, num_pages=160, max_requests=3, max_model_len=640)
    outs, pos, other = [], 0, 0
    for n in cuts:
        entries, rows = [StepEntry("a", [0] * n, [])], [x[pos:pos + n]]
        if batch_with is not None and other < batch_with.shape[0]:
            m = min(3, batch_with.shape[0] - other)
            entries.insert(0, StepEntry("b", [0] * m, []))
            rows.insert(0, batch_with[other:other + m])
            other += m
        starts = []
        for e in entries:
            if not eng.cache.has_request(e.request_id):
                eng.cache.add_request(e.request_id)
            starts.append(eng.cache.append(e.request_id, len(e.tokens)))
        ctx = eng._build_context(entries, starts)
        inp = torch.cat(rows).to(DEV, rt.dtype).contiguous()
        cache = eng.cache.view(0) if 0 in eng.cache else None
        out = part.forward(ctx, inp, cache) if part.is_mixer else part.forward(ctx, inp)
        out = out.double().sum(0) if out.dim() == 3 else out.double()
        outs.append(out[-n:].cpu().numpy())
        pos += n
    return np.concatenate(outs)


def part_weights(part, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    wt = {}
    for n, s in part.param_specs().items():
        if len(s.shape) == 2:
            wt[n] = (torch.randn(s.shape, generator=g) * scale / math.sqrt(s.shape[1])).to(torch.bfloat16)
        else:
            wt[n] = ((1.0 if s.kind == "norm" else 0.0) + torch.randn(s.shape, generator=g) * (0.1 if s.kind == "norm" else 1.0)).to(torch.bfloat16)
    return wt, {n: t.double().numpy() for n, t in wt.items()}


def rel(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-9))


PART_TOL = {"float32": 2e-5, "bfloat16": 4e-2}
CUTS = (13, 1, 1, 2, 30, 1, 7, 2, 1, 1, 1, 1, 40, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 5)


@pytest.fixture(params=["matrix", "fma"])
def portion_kernel(request):
    """Steps with prompt portions on the matrix-instruction kernel (the default) and on the FMA one."""
    from rustinfer_amd.kernels import ops
    keep, ops.WINDOW_ATTENTION_MFMA = ops.WINDOW_ATTENTION_MFMA, request.param == "matrix"
    yield request.param
    ops.WINDOW_ATTENTION_MFMA = keep


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,dk,dv,rot,window,scale,inter", [
    (4, 2, 16, 24, 8, 9, 0.3, False), (3, 3, 40, 36, 40, 1, 0.2, False), (8, 1, 32, 16, 2, 33, 0.18, True),
    (2, 2, 128, 128, 64, 70, 0.09, False), (5, 5, 72, 200, 72, 17, 0.12, False), (6, 2, 64, 64, 64, 500, 0.125, False),
    (6, 1, 24, 40, 12, 21, 0.2, False), (2, 1, 256, 256, 256, 40, 0.06, False)])
def test_window_attention_alone(dtype, H, G, dk, dv, rot, window, scale, inter, portion_kernel):
    from rustinfer_amd.parts import RotaryEmbedding, WindowAttention
    d = 48
    pe, vpe = RotaryEmbedding(dk, 300.0, rot_dim=rot), RotaryEmbedding(dv, 300.0)
    att = WindowAttention(d, H, G, dk, dv, scale, window=window, pos_enc=pe, value_pos_enc=vpe, interleaved_values=inter)
    wt, w = part_weights(att, H * dk + window, scale=2.0)
    from rustinfer_amd.engine import make_runtime
    att.load(wt, make_runtime(dtype, DEV))
    T = sum(CUTS)
    x = torch.randn(T, d, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).float()
    m = dict(heads=H, kv_heads=G, dim=dk, vdim=dv, mask=dict(size=window), scale=scale, rot=dict(base=300.0, dims=rot))
    if inter:
        ref = interleaved_reference(x.double().numpy(), w, m)
    else:
        ref = P.windowed_attention(x.double().numpy(), w, m)
    got = run_part(att, [pe, vpe], dtype, x, CUTS)
    assert rel(got, ref) < PART_TOL[dtype]


def interleaved_reference(n, w, m):
    """The plain attention with the values' pairs (2m, 2m + 1) instead of (m, m + vdim/2): the same
    function on values whose features are permuted so that the pairs become halves, and back."""
    dv, G, H = m["vdim"], m["kv_heads"], m["heads"]
    perm = np.concatenate([np.arange(0, dv, 2), np.arange(1, dv, 2)])          # halves layout <- interleaved
    wv = w["v"].reshape(G, dv, -1)[:, perm].reshape(G * dv, -1)
    wo = w["o"].reshape(-1, H, dv)[:, :, perm].reshape(-1, H * dv)
    return P.windowed_attention(n, dict(w, v=wv, o=wo), m)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,dk,dv,decay", [(2, 16, 24, [0.9, 0.5]), (3, 72, 40, [0.999, 0.7, 0.2]), (1, 128, 64, [0.95]),
                                           (2, 200, 8, [0.99, 0.6]), (1, 1, 1, [0.5])])
def test_lightning_alone(dtype, H, dk, dv, decay):
    from rustinfer_amd.engine import make_runtime
    from rustinfer_amd.parts import LightningAttention
    d = 40
    mix = LightningAttention(d, H, dk, dv, decay, 1e-5)
    wt, w = part_weights(mix, dk + dv)
    mix.load(wt, make_runtime(dtype, DEV))
    x = torch.randn(sum(CUTS), d, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16).float()
    ref = P.lightning_attention(x.double().numpy(), w, dict(heads=H, dim=dk, vdim=dv, decay=decay), 1e-5)
    other = torch.randn(50, d, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16).float()
    got = run_part(mix, [], dtype, x, CUTS, batch_with=other)
    assert rel(got, ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,dim,rank", [(2, 16, 4), (3, 72, 12), (1, 128, 8), (2, 33, 5), (1, 256, 16)])
def test_general_delta_rule_alone(dtype, H, dim, rank):
    from rustinfer_amd.engine import make_runtime
    from rustinfer_amd.parts import GeneralDeltaRule
    d = 56
    mix = GeneralDeltaRule(d, H, dim, rank, 1e-6)
    wt, w = part_weights(mix, dim + rank)
    mix.load(wt, make_runtime(dtype, DEV))
    x = torch.randn(sum(CUTS), d, generator=torch.Generator().manual_seed(8)).to(torch.bfloat16).float()
    ref = P.general_delta_rule(x.double().numpy(), w, dict(heads=H, dim=dim), 1e-6)
    other = torch.randn(50, d, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).float()
    got = run_part(mix, [], dtype, x, CUTS, batch_with=other)
    assert rel(got, ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_dense_feed_forward_and_capped_head(dtype):
    from types import SimpleNamespace
    from rustinfer_amd.engine import Workspace, make_runtime
    from rustinfer_amd.parts import DenseMLP, Embedding, LMHead
    rt = make_runtime(dtype, DEV)
    g = torch.Generator().manual_seed(3)
    mlp = DenseMLP(40, 52, "relu2")
    wt, w = part_weights(mlp, 1)
    mlp.load(wt, rt)
    x = torch.randn(70, 40, generator=g).to(torch.bfloat16)
    ctx = SimpleNamespace(workspace=Workspace(rt.device))
    out = mlp.forward(ctx, x.to(DEV, rt.dtype))
    out = out.double().sum(0) if out.dim() == 3 else out.double()
    assert rel(out.cpu().numpy(), P.dense_ff(x.double().numpy(), w)) < PART_TOL[dtype]
    table = (torch.randn(90, 40, generator=g)).to(torch.bfloat16)
    emb = Embedding(90, 40, weight_name="")
    emb.load({"": table}, rt)
    head = LMHead(90, 40, tied_to=emb, logit_scale=0.6, softcap=3.0)
    head.load({}, rt)
    logits = torch.empty(70, 90, device=DEV)
    head.forward(None, x.to(DEV, rt.dtype), logits)
    ref = 3.0 * np.tanh(0.6 * (x.double().numpy() @ table.double().numpy().T) / 3.0)
    assert rel(logits.double().cpu().numpy(), ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decoded", [False, True])
def test_one_key_decides_at_the_windows_edge(dtype, decoded, portion_kernel):
    """A query that matches one far key a hundredfold: with the key on the window's last
    position the output is that key's value (turned by the distance), one position further out
    it is not seen at all.  Among 300 keys, across pages, in a prompt and in single tokens."""
    from rustinfer_amd.engine import make_runtime
    from rustinfer_amd.parts import RotaryEmbedding, WindowAttention
    dk, dv, window, T = 16, 12, 37, 300
    d = dk
    pe, vpe = RotaryEmbedding(dk, 100.0, rot_dim=2), RotaryEmbedding(dv, 100.0)
    att = WindowAttention(d, 1, 1, dk, dv, 1.0, window=window, pos_enc=pe, value_pos_enc=vpe)
    g = torch.Generator().manual_seed(1)
    eye = torch.eye(dk)
    wt = {"q": eye, "k": eye, "v": torch.randn(dv, d, generator=g), "o": torch.randn(d, dv, generator=g)}
    wt = {n: t.to(torch.bfloat16) for n, t in wt.items()}
    att.load(wt, make_runtime(dtype, DEV))
    w = {n: t.double().numpy() for n, t in wt.items()}
    x = 0.1 * torch.randn(T, d, generator=g)
    marked, inside, outside = 200, 200 + window - 1, 200 + window
    x[marked] = 0.0
    x[marked, 7] = 8.0                       # feature 7 is not among the rotated ones
    x[marked, 9] = 1.0
    for i in (inside, outside):
        x[i, 7] = 8.0
    x = x.to(torch.bfloat16).float()
    m = dict(heads=1, kv_heads=1, dim=dk, vdim=dv, mask=dict(size=window), scale=1.0, rot=dict(base=100.0, dims=2))
    ref = P.windowed_attention(x.double().numpy(), w, m)
    assert np.abs(ref[inside] - ref[outside]).max() > 0.3 * np.abs(ref[inside]).max()     # the test can tell
    cuts = [150] + [1] * 150 if decoded else [150, 90, 60]
    got = run_part(att, [pe, vpe], dtype, x, cuts, page=16)
    for i in (inside - 1, inside, outside, outside + 1):
        assert rel(got[i], ref[i]) < PART_TOL[dtype], i


# ---------------------------------------------------------------------------
# whole models through the engine's step function
# ---------------------------------------------------------------------------
LENGTHS = (70, 3, 121, 1, 38)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_every_cut_gives_the_plain_logits(tdirs, plain_logits, name, dtype):
    reqs, logits = plain_logits(name, LENGTHS, 21)
    eng = engine_for(tdirs[name], dtype, name)
    for label, steps in (("whole", cut_whole(reqs)), ("last tokens alone", cut_tail_single(reqs, tail=50)),
                         ("portions", cut_portions(reqs, seed=3)),
                         ("portions of two", cut_portions(reqs, seed=4, sizes=(2, 2, 3, 2, 1, 2)))):
        check_rows(steps, run_steps(eng, steps), logits, dtype, f"{name} {dtype} {label}")
        assert not eng.cache.live_requests()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_mixed_batches_with_pages_and_slots_used_again(tdirs, plain_logits, name, dtype):
    lengths = (90, 17, 64, 5, 130, 33, 2, 71)
    reqs, logits = plain_logits(name, lengths, 22)
    page = PAGE[name]
    max_tokens = 3 * (-(-130 // 64) * 64)
    eng = engine_for(tdirs[name], dtype, name, num_pages=max_tokens // page, max_requests=3, max_len=256)
    steps = cut_mixed(reqs, max_tokens, seed=5, max_live=3, tail=6)
    assert max(len(st["entries"]) for st in steps) == 3
    slots = set()
    results = {}
    from rustinfer_amd.engine import StepEntry
    for st in steps:
        lg = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]])
        slots.update(eng.cache.slot(e["id"]) for e in st["entries"])
        if lg.shape[0]:
            results[st["step"]] = lg.cpu().numpy()
        for rid in st["end"]:
            eng.release(rid)
    assert len(slots) == 3 and len(reqs) > 3             # eight requests went through three state slots
    check_rows(steps, results, logits, dtype, f"{name} {dtype} mixed")
    eng.cache.check()


@pytest.mark.parametrize("name", ["P", "Q"])
def test_a_batch_gives_what_each_request_gives_alone(tdirs, name):
    from rustinfer_amd.engine import StepEntry
    cfg = CONFIGS[name]
    reqs = random_requests(cfg["vocab"], (40, 9, 1, 25), 30)
    eng = engine_for(tdirs[name], "float32", name)
    alone = {}
    for rid, toks in reqs.items():
        if len(toks) > 1:
            eng.step([StepEntry(rid, toks[:-1], [])])
        alone[rid] = eng.step([StepEntry(rid, toks[-1:], [0])]).cpu().numpy()[0]
        eng.release(rid)
    first = [StepEntry(rid, toks[:-1], []) for rid, toks in reqs.items() if len(toks) > 1]
    eng.step(first)
    both = eng.step([StepEntry(rid, toks[-1:], [0]) for rid, toks in reqs.items()]).cpu().numpy()
    s = float(np.std(both))
    for row, rid in enumerate(reqs):
        assert np.abs(both[row] - alone[rid]).max() < 1e-4 * s, rid


@pytest.mark.parametrize("name", ["P", "Q"])
def test_long_decoding(tdirs, plain, name):
    """Twenty tokens of prompt and 280 single tokens: the window passes over decoded tokens, pages
    are given back on the way, the state is carried 280 times."""
    cfg, w = plain[name]
    toks = random_requests(cfg["vocab"], (300,), 40)["r0"]
    logits = {"r0": P.forward(cfg, w, toks)}
    eng = engine_for(tdirs[name], "float32", name, num_pages=32)
    steps = cut_tail_single({"r0": toks}, tail=280)
    check_rows(steps, run_steps(eng, steps), logits, "float32", f"{name} long decoding")


@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_scheduler(tdirs, plain, name):
    from rustinfer_amd.llm import LLM
    from rustinfer_amd.sampling import SamplingParams
    cfg, w = plain[name]
    prompts = list(random_requests(cfg["vocab"], (12, 47, 5, 30, 21), 50).values())
    llm = LLM(model=tdirs[name], dtype="float32", paged_block_size=PAGE[name], num_blocks=48, max_batch_seqs=3,
              max_model_len=128, max_batch_tokens=64, chunked_prefill_size=32)
    res = llm.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    for p, r in zip(prompts, res):
        assert len(r.token_ids) == 12
        toks = list(p)
        for i, t in enumerate(r.token_ids):
            row = P.forward(cfg, w, toks)[-1]
            assert row.max() - row[t] < 1e-3 * max(1.0, float(np.std(row))), (i, t, int(np.argmax(row)))
            toks.append(t)
    assert llm.engine.graph_replays > 0 or not llm.engine._graph_sizes


def test_trace_replay_of_a_tedelix_model(tdirs, plain_logits, tmp_path):
    """bin/trace_run as a user starts it, on the mixed cut, four state slots."""
    import subprocess
    import sys
    from helpers import ROOT
    name = "P"
    reqs, logits = plain_logits(name, (50, 20, 9, 77, 30), 60)
    steps = cut_mixed(reqs, 512, seed=1, max_live=4, tail=5)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", tdirs[name], "--dtype", "float32",
           "--out", str(tmp_path), "--max-tokens", "512"]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {st['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    results = {}
    for st in steps:
        n = sum(len(e["want"]) for e in st["entries"])
        if n:
            results[st["step"]] = np.fromfile(os.path.join(str(tmp_path), f"{st['step']}.f32"), dtype="<f4").reshape(n, -1)
    check_rows(steps, results, logits, "float32", "trace replay")
