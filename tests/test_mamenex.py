"""Mamenex on the host: its configuration, the model it describes, what its layers ask of the cache manager, and the
plain implementation's mechanisms against each other."""
import math

import pytest
import torch

import mamenex_models
import plain_mamenex as plain


def _describe(config):
    from bare_cuda_4gib_amd.config.registry import architecture_for
    arch = architecture_for(config)
    return arch, arch.config_class.from_dict(config)


def test_the_architecture_is_chosen_by_its_name():
    arch, cfg = _describe(mamenex_models.CONFIGS["P"])
    assert arch.name == "Mamenex" and cfg.vocab_size == 96 and cfg.hidden_size == 48 and cfg.canon_taps == 2
    assert cfg.norm_eps == 1e-6 and len(cfg.layers) == 4


@pytest.mark.parametrize("name", sorted(mamenex_models.CONFIGS))
def test_the_model_asks_for_exactly_the_tensors_of_the_design(name):
    from bare_cuda_4gib_amd.engine import Model
    config = mamenex_models.CONFIGS[name]
    arch, cfg = _describe(config)
    expected = {n: s for n, s in Model(arch.describe(cfg)).expected_weights().items() if not s.optional}
    drawn = mamenex_models.tensors_for(config, 1)
    assert set(expected) == set(drawn)
    for n, spec in expected.items():
        assert tuple(spec.shape) == tuple(drawn[n].shape), n
    # a layer without a feed-forward has neither its tensors nor its norms
    for n, layer in enumerate(config["layers"]):
        assert (f"l{n}.norm2" in expected) == (layer["mlp"] is not None) == (f"l{n}.mlp.up" in expected)


def test_what_is_refused():
    from bare_cuda_4gib_amd.errors import ConfigError
    base = mamenex_models.CONFIGS["R"]

    def broken(change):
        import copy
        c = copy.deepcopy(base)
        change(c)
        return c
    for change in (lambda c: c["layers"][0].update(type="lstm"),
                   lambda c: c["layers"][1]["mixer"].pop("kv_rank"),
                   lambda c: c["layers"][0].update(mlp=dict(kind="routed", ff=8)),
                   lambda c: c["canon"].update(taps=0),
                   lambda c: c.pop("norm"),
                   lambda c: c["layers"][0]["mixer"].update(blocks=5),          # 36 channels in 5 blocks
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3)):
        with pytest.raises(ConfigError):
            arch, cfg = _describe(broken(change))
            from bare_cuda_4gib_amd.engine import Model
            Model(arch.describe(cfg))


def test_a_layer_keeps_its_mixers_cache_and_the_tail_of_its_input_convolution():
    from bare_cuda_4gib_amd.cache import CacheManager, PagedLatent
    from bare_cuda_4gib_amd.engine import Model
    arch, cfg = _describe(mamenex_models.CONFIGS["P"])
    streams = Model(arch.describe(cfg)).cache_streams()
    assert dict(streams[1].members)["mixer"] == PagedLatent(20, 12, 0)
    cm = CacheManager(streams, page_tokens=4, num_pages=6, max_requests=2, max_tokens=24, dtype=torch.float32, device="cpu")
    assert list(cm.groups) == [("window", 0)]                 # the two attention layers share one pool
    v = cm.view(0)
    assert tuple(v.mixer.state.shape) == (3, 40) and v.mixer.state.dtype == torch.float32
    assert tuple(v.mixer.tail.shape) == (3, 2, 40) and tuple(v.conv.tail.shape) == (3, 1, 48)
    assert tuple(cm.view(1).mixer.latent.shape) == (7, 4, 32) and cm.view(1).mixer.group == ("window", 0)
    assert tuple(cm.view(3).mixer.tail.shape) == (3, 0, 24)   # a convolution of one tap has no tail
    # state is zeroed at admission, also in a slot that another request has used
    a = cm.admit("a")
    v.mixer.state[a] = 7.0
    v.conv.tail[a] = 7.0
    saved = cm.save_slots([a])
    v.mixer.state[a] = 9.0
    cm.restore_slots(saved)
    assert float(v.mixer.state[a].min()) == 7.0
    cm.release("a")
    assert cm.admit("b") == a and float(v.mixer.state[a].abs().max()) == 0.0 and float(v.conv.tail[a].abs().max()) == 0.0


# ---- the plain implementation's mechanisms, each against a second way of writing it ----

def test_plain_convolution_is_causal_and_its_last_column_is_the_current_token():
    v = torch.randn(9, 3, dtype=torch.float64)
    w = torch.randn(3, 4, dtype=torch.float64)
    out = plain.causal_conv(v, w)
    assert torch.allclose(out[0], w[:, 3] * v[0])
    assert torch.allclose(out[5], w[:, 3] * v[5] + w[:, 2] * v[4] + w[:, 1] * v[3] + w[:, 0] * v[2])


def test_plain_rotation_turns_neighbouring_pairs_and_leaves_the_rest():
    v = torch.randn(5, 2, 6, dtype=torch.float64)
    pos = torch.arange(5)
    out = plain.interleaved_rotation(v, pos, 100.0, 4)
    assert torch.equal(out[..., 4:], v[..., 4:]) and torch.allclose(out[0], v[0])
    ang = 3 * 100.0 ** (-2.0 / 4)
    assert torch.allclose(out[3, 1, 2], v[3, 1, 2] * math.cos(ang) - v[3, 1, 3] * math.sin(ang))
    assert torch.allclose(out[3, 1, 3], v[3, 1, 3] * math.cos(ang) + v[3, 1, 2] * math.sin(ang))
    assert torch.allclose(out.norm(dim=-1), v.norm(dim=-1))


def test_plain_sink_takes_weight_without_a_value():
    s = torch.tensor([0.3, -1.0, 2.0], dtype=torch.float64)
    w = plain.sink_softmax(s, 1.5)
    assert math.isclose(float(w.sum()), float(torch.exp(s).sum() / (torch.exp(s).sum() + math.exp(1.5))))
    assert torch.allclose(plain.sink_softmax(s, -1e9), torch.softmax(s, 0))


def test_plain_activation_is_smooth_at_zero():
    p, q = torch.tensor(0.3, dtype=torch.float64), torch.tensor(-0.4, dtype=torch.float64)
    z = torch.tensor([-1e-7, 0.0, 1e-7], dtype=torch.float64)
    a = plain.xielu(z, p, q)
    assert abs(float(a[1])) == 0.0 and abs(float(a[2] - a[0]) / 2e-7 - 0.5) < 1e-6


def test_plain_latent_attention_equals_attention_with_the_up_projections_absorbed():
    """Scores against the latent with Wuk^T q, values up-projected after the weighted sum: the same numbers."""
    torch.manual_seed(0)
    m = mamenex_models.latent(2, 6, 4, 5, 7, dims=4)["mixer"]
    T, W, H, dn, dr, dv, r = 6, 12, 2, 6, 4, 5, 7
    w = {k: v.double() for k, v in mamenex_models.tensors_for(dict(vocab=5, width=W, canon=dict(taps=1), layers=[
        dict(type="latent_attention", mixer=m, mlp=None)]), 3).items()}
    w = {k[len("l0.mix."):]: v for k, v in w.items() if k.startswith("l0.mix.")}
    h = torch.randn(T, W, dtype=torch.float64)
    want = plain.latent_attention(h, w, m, 1e-6)
    pos = torch.arange(T)
    q = (h @ w["q"].T).view(T, H, dn + dr)
    dkv = h @ w["dkv"].T
    c = plain.plain_rmsnorm(dkv[:, :r], w["dkv.norm"], 1e-6)
    kr = plain.interleaved_rotation(dkv[:, r:], pos, m["rot"]["base"], 4)
    qr = plain.interleaved_rotation(q[..., dn:], pos, m["rot"]["base"], 4)
    out = torch.zeros(T, H, dv, dtype=torch.float64)
    for a in range(H):
        q_abs = q[:, a, :dn] @ w["uk"].view(H, dn, r)[a]                 # [T, r]
        for t in range(T):
            s = (c[:t + 1] @ q_abs[t] + kr[:t + 1] @ qr[t, a]) * m["scale"]
            out[t, a] = w["uv"].view(H, dv, r)[a] @ (plain.sink_softmax(s, w["sink"][a]) @ c[:t + 1])
    assert torch.allclose(out.reshape(T, H * dv) @ w["o"].T, want, atol=1e-12)


def test_plain_model_runs_every_configuration():
    for name, config in mamenex_models.CONFIGS.items():
        w = mamenex_models.tensors_for(config, 5)
        layers = []
        logits = plain.forward(config, w, [1, 2, 3, 4, 5, 6, 7], layer_outputs=layers)
        assert tuple(logits.shape) == (7, config["vocab"]) and len(layers) == len(config["layers"])
        assert bool(torch.isfinite(logits).all())
        # causal: a later token changes nothing before it
        again = plain.forward(config, w, [1, 2, 3, 4, 9, 6, 7])
        assert torch.equal(again[:4], logits[:4]) and not torch.allclose(again[4:], logits[4:])
