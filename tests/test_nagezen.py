"""Nagezen on the host: its configuration, the model it describes, what its layers ask of the cache manager (the
kept first tokens beside a window), and the plain implementation's mechanisms against each other."""
import copy
import math

import pytest
import torch

import nagezen_models
import plain_nagezen as plain


def _describe(config):
    from bare_cuda_4gib_amd.config.registry import architecture_for
    arch = architecture_for(config)
    return arch, arch.config_class.from_dict(config)


def test_the_architecture_is_chosen_by_its_name():
    arch, cfg = _describe(nagezen_models.CONFIGS["A"])
    assert arch.name == "Nagezen" and cfg.vocab_size == 96 and cfg.hidden_size == 48 and cfg.streams == 2
    assert cfg.norm_eps == 1e-5 and cfg.logit_scale == 1.5 and len(cfg.layers) == 4
    spec = arch.describe(cfg)
    assert spec.streams == 2 and [l.block for l in spec.layers] == ["hyper"] * 4
    assert [l.mixer.kind for l in spec.layers] == ["retention", "diff_attention", "gla", "diff_attention"]
    assert spec.layers[1].mixer.params["window"] == 9 and spec.layers[1].mixer.params["keep_first"] == 3
    assert spec.layers[1].mixer.params["position"].params["scaling"]["factor"] == 8.0
    assert spec.layers[2].ffn is None and "ffn_conn" not in spec.layers[2].extras
    assert spec.final_norm.params["out_scale"] == 1.5


@pytest.mark.parametrize("name", sorted(nagezen_models.CONFIGS))
def test_the_model_asks_for_exactly_the_tensors_of_the_design(name):
    from bare_cuda_4gib_amd.engine import Model
    config = nagezen_models.CONFIGS[name]
    arch, cfg = _describe(config)
    expected = Model(arch.describe(cfg)).expected_weights()
    drawn = nagezen_models.tensors_for(config, 1)
    assert set(expected) == set(drawn)
    for n, spec in expected.items():
        assert tuple(spec.shape) == tuple(drawn[n].shape), n
    for n, layer in enumerate(config["layers"]):
        assert (f"l{n}.norm2" in expected) == (layer["mlp"] is not None) == (f"l{n}.hc2.mix" in expected)
    # without the rank in the configuration the decay map's tensors say it: any size is taken there
    bare = copy.deepcopy(config)
    for layer in bare["layers"]:
        layer["mixer"].pop("rank", None)
    arch, cfg = _describe(bare)
    for n, spec in Model(arch.describe(cfg)).expected_weights().items():
        if n.endswith("mix.a1") or n.endswith("mix.a2"):
            assert -1 in spec.shape
        else:
            assert tuple(spec.shape) == tuple(drawn[n].shape), n


def test_what_is_refused():
    from bare_cuda_4gib_amd.engine import Model
    from bare_cuda_4gib_amd.errors import ConfigError
    base = nagezen_models.CONFIGS["A"]

    def broken(change):
        c = copy.deepcopy(base)
        change(c)
        return c
    for change in (lambda c: c["layers"][0].update(type="lstm"),
                   lambda c: c["layers"][1]["mixer"].pop("kv_heads"),
                   lambda c: c["layers"][1]["mixer"].update(kv_heads=3),           # four heads on three key/value heads
                   lambda c: c["layers"][0].update(mlp=dict(kind="routed", ff=8, limit=1.0)),
                   lambda c: c["layers"][0]["mlp"].pop("limit"),
                   lambda c: c["layers"][0]["mixer"].update(decay=[0.5, 0.5]),      # three heads, two decays
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=14),        # more than a map has
                   lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("slow"),
                   lambda c: c["layers"][2]["mixer"].update(tau=0.0),
                   lambda c: c.update(streams=17),
                   lambda c: c.pop("norm")):
        with pytest.raises(ConfigError):
            arch, cfg = _describe(broken(change))
            Model(arch.describe(cfg))


def test_what_the_layers_keep():
    from bare_cuda_4gib_amd.cache.specs import FixedState, PagedHeads
    from bare_cuda_4gib_amd.engine import Model
    arch, cfg = _describe(nagezen_models.CONFIGS["A"])
    streams = Model(arch.describe(cfg)).cache_streams()
    assert streams[0] == FixedState((3, 8, 12), "float32") and streams[2] == FixedState((2, 16, 10), "float32")
    assert streams[1] == PagedHeads(4, 12, 2, 20, 9, 3) and streams[3] == PagedHeads(6, 10, 3, 6, 11, 0)
    assert streams[1].group_key() != streams[3].group_key()
    assert PagedHeads(2, 4, 1, 4).group_key() == ("window", 0) and PagedHeads(2, 4, 1, 4, 0, 5).always_kept() == 0


def test_kept_first_tokens_stay_while_the_window_gives_pages_back():
    """Window 6 with 5 kept first tokens over pages of 4: the two pages that hold the kept tokens are never given back,
    the pages between them and the window are, and the peak a scheduler plans with counts both."""
    from bare_cuda_4gib_amd.cache.manager import CacheManager
    from bare_cuda_4gib_amd.cache.specs import PagedHeads
    spec = PagedHeads(2, 4, 1, 4, window=6, keep_first=5)
    cm = CacheManager({"a": spec, "plain": PagedHeads(2, 4, 1, 4, window=6)}, page_tokens=4, num_pages=12, max_requests=2,
                      max_tokens=64, dtype=torch.float32, device="cpu")
    key = spec.group_key()
    assert set(cm.groups) == {key, ("window", 6)}
    cm.admit("r")
    length = 0
    for n in (3, 4, 2, 8, 1, 5, 9, 1, 1, 7):
        cm.reserve([("r", n)])
        # every key that a row of this step reads lies in a page the request still holds
        table = cm.table(key, "r")
        for pos in range(length, length + n):
            for j in range(pos + 1):
                if pos - j < 6 or j < 5:
                    assert table[j // 4] >= 0, (pos, j)
        cm.advance("r", n)
        length += n
        table, other = cm.table(key, "r"), cm.table(("window", 6), "r")
        first = max(0, length - 5) // 4
        assert [p >= 0 for p in table] == [i < 2 or i >= first for i in range(len(table))], f"after {length} tokens"
        assert [p >= 0 for p in other] == [i >= first for i in range(len(other))]
    peak = cm.peak_pages(64, 5)
    assert peak[key] == peak[("window", 6)] + 2
    most = max(sum(1 for p in cm.table(key, "r") if p >= 0), 0)
    assert most <= peak[key]
    cm.release("r")
    assert cm.pages_in_use() == 0


def test_the_plain_mechanisms_against_each_other():
    """The state form of linear attention equals its sum form; the rotation leaves the products of a query and a key
    depending on their distance alone (scaled or not); a window as wide as the sequence is no window."""
    torch.manual_seed(0)
    T, d, e = 12, 6, 5
    q, k, v = (torch.randn(T, d, dtype=torch.float64), torch.randn(T, d, dtype=torch.float64), torch.randn(T, e, dtype=torch.float64))
    decay = torch.rand(T, d, dtype=torch.float64) * 0.5 + 0.5
    got = plain.decayed_outer_products(q, k, v, decay)
    for t in range(T):
        want = torch.zeros(e, dtype=torch.float64)
        for j in range(t + 1):
            w = torch.prod(decay[j + 1:t + 1], dim=0)
            want += float((q[t] * w * k[j]).sum()) * v[j]
        assert torch.allclose(got[t], want, atol=1e-12)
    scaling = dict(factor=4.0, original=32, fast=8.0, slow=1.0)
    for sc in (None, scaling):
        a, b = torch.randn(1, 8, dtype=torch.float64), torch.randn(1, 8, dtype=torch.float64)
        dots = []
        for p in (0, 100):
            ca, sa = plain.half_rotation_angles(torch.tensor([p + 7]), 6, 100.0, sc)
            cb, sb = plain.half_rotation_angles(torch.tensor([p]), 6, 100.0, sc)
            dots.append(float((plain.half_rotation(a, ca, sa) * plain.half_rotation(b, cb, sb)).sum()))
        assert math.isclose(dots[0], dots[1], rel_tol=1e-9, abs_tol=1e-9)
    assert all(plain.visible(9, j, 10, 0) for j in range(10)) and not plain.visible(10, 0, 10, 0) and plain.visible(10, 0, 10, 1)
    assert not plain.visible(3, 4, 0, 0) and plain.visible(400, 0, 0, 0)
