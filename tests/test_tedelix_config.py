"""Tedelix without a GPU: its configuration reader, the registry, the tensors the model asks
for, the size that only the checkpoint gives, the random-weights writer read back by the plain
implementation's own reader, and the cache books for value heads of another size than key heads."""
import json
import os

import pytest
import torch

import plain_tedelix as P
from rustinfer_amd.config import (ConfigError, GeneralDeltaSpec, LightningSpec, TedelixConfig, WindowAttentionSpec,
                                  load_model_config, resolve_architecture)

CFG = dict(architecture="Tedelix", vocab=150, width=48, norm=dict(eps=1e-5), logit_scale=0.8, logit_softcap=20.0, layers=[
    dict(type="lightning", mixer=dict(heads=2, dim=8, vdim=12, decay=[0.9, 0.6]), mlp=dict(kind="dense", ff=32)),
    dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=8, vdim=10, mask=dict(size=7), scale=0.4,
                                      rot=dict(base=100.0, dims=4)), mlp=None),
    dict(type="general_delta", mixer=dict(heads=3, dim=8), mlp=dict(kind="dense", ff=16)),
])


def test_reads_every_size_and_constant():
    cfg = TedelixConfig.from_dict(CFG)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.logit_scale, cfg.logit_softcap) == (150, 48, 1e-5, 0.8, 20.0)
    l, a, g = (layer.mixer for layer in cfg.layers)
    assert isinstance(l, LightningSpec) and (l.heads, l.dim, l.vdim, l.decay) == (2, 8, 12, (0.9, 0.6))
    assert isinstance(a, WindowAttentionSpec) and (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.rot_base, a.rot_dims, a.scale) \
        == (4, 2, 8, 10, 7, 100.0, 4, 0.4)
    assert isinstance(g, GeneralDeltaSpec) and (g.heads, g.dim, g.decay_rank) == (3, 8, None)
    assert [layer.ff for layer in cfg.layers] == [32, None, 16]
    assert cfg.eos_token_ids == ()
    assert TedelixConfig.from_dict(cfg.to_dict()) == cfg
    assert resolve_architecture(CFG).name == "Tedelix"


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("vocab"), "vocab"), (lambda c: c.update(layers=[]), "layers"),
    (lambda c: c["layers"][0].update(type="conv"), "unknown mixer"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3), "even"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][2].update(mlp=dict(kind="experts", ff=8)), "dense"),
    (lambda c: c["norm"].pop("eps"), "eps")])
def test_refuses_what_it_cannot_run(change, word):
    bad = json.loads(json.dumps(CFG))
    change(bad)
    with pytest.raises(ConfigError, match=word):
        TedelixConfig.from_dict(bad)


def test_model_asks_for_the_designs_tensors_and_rank_comes_from_the_checkpoint(tmp_path):
    from rustinfer_amd.config import TedelixLayer
    from rustinfer_amd.weights import write_random_model
    cfg = TedelixConfig.from_dict(CFG)
    layers = list(cfg.layers)
    layers[2] = TedelixLayer(GeneralDeltaSpec(3, 8, decay_rank=5), layers[2].ff)
    cfg5 = TedelixConfig(**{**cfg.__dict__, "layers": tuple(layers)})
    d = write_random_model(cfg5, 3, str(tmp_path))
    entry, read = load_model_config(d)
    assert "decay_rank" not in json.dumps(json.load(open(os.path.join(d, "config.json"))))
    assert read.layers[2].mixer.decay_rank == 5          # from the shape of l2.mix.w1
    specs = entry.builder(read).param_specs()
    pcfg, w = P.read_model(d)                            # the plain reader sees the same names and shapes
    assert {n: tuple(s.shape) for n, s in specs.items()} == {n: a.shape for n, a in w.items()}
    assert sorted(n for n in specs if n.startswith("l2.")) == sorted(
        "l2." + n for n in ("norm1", "mix.r", "mix.k", "mix.v", "mix.g", "mix.a", "mix.a.b", "mix.w1", "mix.w2", "mix.w0",
                            "mix.norm", "mix.o", "mlp.up", "mlp.down"))
    assert {"embed", "final.norm", "l0.mix.norm", "l1.mix.q", "l1.mix.o"} <= set(specs) and "l1.mlp.up" not in specs
    assert specs["l1.mix.v"].shape == (2 * 10, 48) and specs["l2.mix.w1"].shape == (5, 48)
    logits = P.forward(pcfg, w, [1, 2, 3])               # and the plain implementation runs it
    assert logits.shape == (3, 150) and abs(logits).max() <= 20.0


def test_cache_needs_and_books_for_value_heads_of_another_size():
    from rustinfer_amd.cache.manager import CacheManager
    from rustinfer_amd.parts import PagedKVNeed, StateNeed
    model = resolve_architecture(CFG).builder(TedelixConfig.from_dict(CFG))
    needs = model.cache_needs()
    assert needs == {0: StateNeed((2, 8, 12), torch.float32), 1: PagedKVNeed(2, 8, 7, 10), 2: StateNeed((3, 8, 8), torch.float32)}
    cm = CacheManager(needs, page_size=4, num_pages=6, max_requests=2, max_model_len=64)
    cm.add_request("a")
    cm.append("a", 9)
    assert cm.table(0, "a") == [0, 1, 2]
    cm.append("a", 11)
    cm.append("a", 1)                                     # a query at position 20 sees keys 14..20: pages 0 to 2 go back
    assert cm.table(0, "a") == [-1, -1, -1, 3, 4, 0] and cm.pages_held("a") == 3
    cm.check()
    cm.release("a")
    cm.add_request("b")
    assert cm.slot("b") == 0                              # the slot is used again
    assert PagedKVNeed(2, 8).value_dim == 8 and PagedKVNeed(2, 8, None, 10).value_dim == 10


def test_bare_tensor_names_reach_their_parts():
    from rustinfer_amd.parts.base import LazyTensors, join_name, narrow_tensors
    t = {"final.norm": 1, "l0.norm1": 2, "l0.mix.a.b": 3, "l0.mix.a": 4, "embed": 5}
    assert narrow_tensors(t, "final.norm") == {"": 1}
    assert narrow_tensors(narrow_tensors(t, "l0"), "mix") == {"a.b": 3, "a": 4}
    lazy = LazyTensors(set(t), lambda n: t[n])
    assert lazy.narrow("embed")[""] == 5 and lazy.narrow("l0").narrow("mix")["a.b"] == 3
    assert sorted(lazy.narrow("l0").keys()) == ["mix.a", "mix.a.b", "norm1"]
    assert join_name("l0", "") == "l0" and join_name("", "x") == "x" and join_name("l0", "mix.q") == "l0.mix.q"
