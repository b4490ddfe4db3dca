"""Begopel without a GPU: its configuration and registry entry, the order of layer runs, the
distance table as the attention part expands it against the plain model's row function, and what
pins the plain model itself (special cases with a closed form)."""
import copy
import math

import numpy as np
import pytest
import torch

import begopel_tiny as bt
from plain import begopel_plain as P


def test_registry_finds_the_architecture_by_either_key():
    from picolm_amd.config import BegopelConfig, resolve
    cfg = bt.CONFIGS["P"]
    assert resolve(cfg).name == "Begopel"
    assert resolve({**cfg, "architectures": ["Begopel"]}).name == "Begopel"
    typed = resolve(cfg).parse_config(cfg)
    assert isinstance(typed, BegopelConfig)
    again = BegopelConfig.from_dict(typed.to_dict())
    assert again == typed


def test_configuration_names_the_faulty_key():
    from picolm_amd.config import BegopelConfig, ConfigError
    base = bt.CONFIGS["P"]

    def broken(path, value):
        c = copy.deepcopy(base)
        d = c
        for k in path[:-1]:
            d = d[k]
        if value is KeyError:
            del d[path[-1]]
        else:
            d[path[-1]] = value
        return c
    cases = [(("width",), KeyError, "width"), (("vocab",), 0, "vocab"), (("layers", 0, "type"), "conv", "layers[0].type"),
             (("layers", 0, "mixer", "left", "kv_heads"), 3, "layers[0].mixer.left.kv_heads"),
             (("layers", 0, "mixer", "right", "conv"), 40, "layers[0].mixer.right.conv"),
             (("layers", 1, "mixer", "groups"), 3, "layers[1].mixer.groups"),
             (("layers", 1, "mixer", "norm_groups"), 5, "layers[1].mixer.norm_groups"),
             (("layers", 1, "mixer", "state"), 1000, "layers[1].mixer.state"),
             (("layers", 2, "mlp", "kind"), "routed", "layers[2].mlp.kind"), (("loop", "stop"), 9, "loop"),
             (("loop", "times"), 0, "loop.times"), (("norm", "eps"), 0.0, "norm.eps")]
    for path, value, named in cases:
        with pytest.raises(ConfigError) as e:
            BegopelConfig.from_dict(broken(path, value))
        assert named in str(e.value), (path, str(e.value))


def test_layer_runs_and_the_models_calls():
    from picolm_amd.config import BegopelConfig
    from picolm_amd.engine.builder import build_from_config_dict
    for cfg in bt.CONFIGS.values():
        typed = BegopelConfig.from_dict(cfg)
        assert typed.layer_runs() == P.layer_runs(cfg)
        model = build_from_config_dict(cfg)
        n = len(cfg["layers"])
        layers_called = [c.block for c in model.order if c.block < n]
        assert layers_called == [i for i, _, _ in P.layer_runs(cfg)]
        entries = [c.block - n for c in model.order if c.block >= n]
        assert entries == list(range(cfg["loop"]["times"])) if cfg.get("loop") else entries == []
        # every run of a layer has a cache entry and a state entry of its own
        seen = set()
        for call, binding in zip(model.order, model.bindings):
            if call.block < n:
                assert binding.writes and (binding.kv, binding.state) not in seen
                seen.add((binding.kv, binding.state))
    assert P.layer_runs(bt.CONFIGS["Q"]) == [(0, None, False), (1, 0, True), (1, 1, True), (1, 2, True), (2, None, False)]


@pytest.mark.parametrize("rows,far", [(8, 40.0), (6, 17.5), (32, 120.0), (2, 3.0), (20, 1000.0)])
def test_distance_rows_are_the_plain_models(rows, far):
    from picolm_amd.parts.sink_attention import distance_rows
    table = distance_rows(rows, far)
    assert len(table) == math.ceil(far) + 1
    for n in range(0, int(far) * 3):
        assert table[min(n, len(table) - 1)] == P.distance_bucket(n, rows, far), n
    assert table[0] == 0 and table[-1] == rows - 1
    assert all(a <= b for a, b in zip(table, table[1:]))


# ------------------------------------------------------------------------------ the plain model itself
def test_plain_attention_special_cases():
    """Without bias, with a sink of minus infinity's stand-in and an open gate, the attention is a
    causal softmax; a sink far above the scores takes all the weight."""
    torch.manual_seed(0)
    T, D, H, G, d, dv = 7, 10, 4, 2, 6, 5
    cfg = dict(heads=H, kv_heads=G, dim=d, vdim=dv, scale=0.37, bias_max=9.0)
    r = lambda *s: torch.randn(*s, dtype=torch.float64)
    W = {"q": r(H * d, D), "k": r(G * d, D), "v": r(G * dv, D), "q.norm": torch.ones(d, dtype=torch.float64),
         "k.norm": torch.ones(d, dtype=torch.float64), "rel": torch.zeros(4, H, dtype=torch.float64),
         "sink": torch.full((H,), -1e9, dtype=torch.float64), "g": torch.zeros(H * dv, D, dtype=torch.float64),
         "o": torch.eye(H * dv, dtype=torch.float64)}
    h = r(T, D)
    got = P.sink_attention(h, W, cfg, 0.0)
    q = P.rms((h @ W["q"].T).view(T, H, d), 0.0)
    k = P.rms((h @ W["k"].T).view(T, G, d), 0.0).repeat_interleave(H // G, dim=1)
    v = (h @ W["v"].T).view(T, G, dv).repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * 0.37
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    want = 0.5 * torch.einsum("hij,jhc->ihc", torch.softmax(s, -1), v).reshape(T, H * dv)       # sigmoid(0) = 1/2
    assert torch.allclose(got, want, atol=1e-12)
    W["sink"] = torch.full((H,), 60.0, dtype=torch.float64)
    assert P.sink_attention(h, W, cfg, 0.0).abs().max() < 1e-12
    # a sink of zero with one key of score zero: the key gets half
    W["sink"] = torch.zeros(H, dtype=torch.float64)
    W["q"] = torch.zeros_like(W["q"])
    first = P.sink_attention(h, W, cfg, 1.0)[0]             # (an eps that keeps the norm of a zero query finite)
    assert torch.allclose(first, 0.5 * 0.5 * v[0].reshape(-1), atol=1e-12)


def test_plain_short_convolution_and_bucket():
    x = torch.arange(12, dtype=torch.float64).view(6, 2)
    w = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)       # column taps-1 multiplies x[t]
    y = P.short_conv(x, w)
    assert y[:, 1].tolist() == x[:, 1].tolist()
    assert y[0, 0] == 0.0 and y[1, 0] == 100.0 * 2 + 10.0 * 0 and y[3, 0] == 100.0 * 6 + 10.0 * 4 + 1.0 * 2
    assert [P.distance_bucket(n, 8, 40.0) for n in (0, 1, 3, 4, 5, 7, 8, 22, 23, 40, 500)] == [0, 1, 3, 4, 4, 4, 5, 6, 7, 7, 7]


def test_plain_delta_rule_and_state_space_recurrences():
    """With a decay of one and a strength of one the delta rule stores v under a unit key exactly: the
    read-out with the same key returns v.  With B = C = a one-hot and no decay the state-space layer
    sums dt x over time."""
    S = torch.zeros(3, 2, dtype=torch.float64)
    k = torch.tensor([0.0, 1.0, 0.0], dtype=torch.float64)
    for v in (torch.tensor([1.0, 2.0], dtype=torch.float64), torch.tensor([-3.0, 5.0], dtype=torch.float64)):
        u = 1.0 * (v - S.T @ k)
        S = S + torch.outer(k, u)
        assert torch.allclose(S.T @ k, v)
    # the same through the mixer's function: one head, identity-like projections
    T, D = 5, 4
    cfg = dict(heads=1, kv_heads=1, dim=2, vdim=2, conv=1)
    z = lambda *s: torch.zeros(*s, dtype=torch.float64)
    W = {"q": z(2, D), "k": z(2, D), "v": z(2, D), "q.conv": torch.ones(2, 1, dtype=torch.float64),
         "k.conv": torch.ones(2, 1, dtype=torch.float64), "v.conv": torch.ones(2, 1, dtype=torch.float64), "b": z(1, D), "a": z(1, D),
         "A_log": torch.tensor([-50.0], dtype=torch.float64), "dt_bias": z(1), "norm": torch.ones(2, dtype=torch.float64),
         "g": z(2, D), "o": torch.eye(2, dtype=torch.float64)}
    W["q"][0, 0] = W["k"][0, 0] = 50.0          # silu(50 h0) is large for h0 > 0: the key is the unit vector e0
    W["v"][0, 1] = W["v"][1, 2] = 1.0
    W["b"][0, 3] = 1.0                          # beta = sigmoid(h3)
    W["g"][:, 3] = 1.0
    h = torch.rand(T, D, dtype=torch.float64) + 0.5
    h[:, 3] = 40.0                              # beta = 1, the gate silu(40) = 40
    out = P.gated_delta(h, W, cfg, 0.0)
    v = P.silu(h[:, 1:3])
    want = P.rms(v * 2 ** -0.5, 0.0) * 40.0     # the read-out is v times the query's length 1/sqrt(dim)
    assert torch.allclose(out, want, rtol=1e-6)


def test_an_unused_second_norm_is_passed_by_and_a_stray_tensor_is_not():
    from picolm_amd.engine.builder import build_from_config_dict
    from picolm_amd.weights import TensorDict, WeightsError, check_specs
    cfg = bt.config(61, 48, [bt.mamba(2, 8, 8, 1, 1, 2, None)])
    w = bt.make_weights(cfg, 0)
    specs = build_from_config_dict(cfg).tensor_specs()
    check_specs(TensorDict(w), specs)
    check_specs(TensorDict({**w, "l0.norm2": torch.zeros(48, dtype=torch.bfloat16)}), specs)
    with pytest.raises(WeightsError) as e:
        check_specs(TensorDict({**w, "l0.norm3": torch.zeros(48, dtype=torch.bfloat16)}), specs)
    assert "l0.norm3" in str(e.value)
    # the distance table's rows are the tensor's to say where the configuration does not name them
    cfg = bt.config(61, 48, [bt.parallel(bt.attention(2, 1, 8, 8, 0.3, 9.0, 4), bt.delta(2, 1, 8, 8, 2), None)])
    w = bt.make_weights(cfg, 0)
    del cfg["layers"][0]["mixer"]["left"]["bias_rows"]
    check_specs(TensorDict(w), build_from_config_dict(cfg).tensor_specs())
