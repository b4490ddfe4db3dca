"""Zarinex without a GPU: the configuration's faults by key, the order of layer runs and their
cache entries, and closed forms that pin the plain model of tests/plain/zarinex_plain.py itself."""
import copy
import math

import numpy as np
import pytest

import zarinex_tiny as zt
from picolm_amd.config import ConfigError, ZarinexConfig, resolve
from picolm_amd.engine.builder import build_from_config_dict
from plain import zarinex_plain as P


def test_the_registry_knows_the_name_and_the_configuration_round_trips():
    for cfg in zt.CONFIGS.values():
        assert resolve(cfg).name == "Zarinex"
        typed = ZarinexConfig.from_dict(cfg)
        assert ZarinexConfig.from_dict(typed.to_dict()) == typed
        assert typed.vocab_size == cfg["vocab"] and typed.hidden_size == cfg["width"]


@pytest.mark.parametrize("path,value,names", [
    (("vocab",), None, "vocab"), (("width",), 0, "width"), (("norm", "eps"), 0.0, "norm.eps"),
    (("layers", 0, "type"), "conv", "layers[0].type"), (("layers", 0, "mixer", "dim"), 300, "layers[0].mixer.dim"),
    (("layers", 2, "mixer", "state"), 1000, "layers[2].mixer.state"), (("layers", 2, "mixer", "conv"), 17, "layers[2].mixer.conv"),
    (("layers", 3, "mixer", "kv_rank"), 2000, "layers[3].mixer.kv_rank"), (("layers", 3, "mixer", "scale"), None, "layers[3].mixer.scale"),
    (("layers", 0, "mlp", "kind"), "dense", "layers[0].mlp.kind"), (("layers", 0, "mlp", "router", "top"), 9, "layers[0].mlp.router.top"),
    (("layers", 3, "mlp", "shared"), 5, "layers[3].mlp.shared"), (("layers", 4, "weights_of"), 4, "layers[4].weights_of"),
    (("layers", 5, "weights_of"), 0, "layers[5].weights_of"), (("layers", 3, "mixer", "scale"), 0.0, "layers[3].mixer.scale"),
    (("layers", 1, "weights_of"), 7, "layers[1].weights_of"),
])
def test_a_fault_names_its_key(path, value, names):
    cfg = copy.deepcopy(zt.CONFIG_A)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        ZarinexConfig.from_dict(cfg)
    assert names in str(e.value)


def test_layer_runs_share_blocks_and_keep_entries_of_their_own():
    model = build_from_config_dict(zt.CONFIG_A)
    # three layers have tensors; six run
    assert len(model.blocks) == 3 and [c.block for c in model.order] == [0, 2, 1, 2, 0, 1]
    kv = [b.kv for b in model.bindings]
    assert kv[1] is not None and kv[3] is not None and kv[1] != kv[3] and kv[0] is None
    states = [b.state for b in model.bindings]
    assert len(set(states)) == 6 and all(s is not None for s in states)          # every run keeps the row before its first
    D, m = 72, zt.CONFIG_A["layers"]
    sizes = {g.shape[0] for g in model.cache_spec.state_groups}
    assert sizes == {D, D + 3 * 24 * 20, D + 2 * 100 + 100 * 12}
    [group] = model.cache_spec.kv_groups
    assert (group.n_entries, group.n_kv_heads, group.head_dim) == (2, 1, 40)      # the latents are the keys, one head of them


def test_a_layer_may_name_one_that_names_another():
    cfg = copy.deepcopy(zt.CONFIG_A)
    cfg["layers"][4]["weights_of"] = 4          # itself
    with pytest.raises(ConfigError):
        ZarinexConfig.from_dict(cfg)
    cfg["layers"].append(copy.deepcopy(cfg["layers"][1]))
    cfg["layers"][4]["weights_of"] = 0
    cfg["layers"][6]["weights_of"] = 1          # which runs with layer 3's
    model = build_from_config_dict(cfg)
    assert [c.block for c in model.order] == [0, 2, 1, 2, 0, 1, 2]


def test_the_plain_positions():
    pe = P.position_rows([0, 3], 6)
    assert np.allclose(pe[0], [0, 1, 0, 1, 0, 1])
    assert np.allclose(pe[1], [math.sin(3), math.cos(3), math.sin(3 * 10000 ** (-2 / 6)), math.cos(3 * 10000 ** (-2 / 6)),
                               math.sin(3 * 10000 ** (-4 / 6)), math.cos(3 * 10000 ** (-4 / 6))])


def test_the_plain_token_shift_and_convolution():
    h = np.arange(6.0).reshape(3, 2) + 1
    assert np.allclose(P.token_shift(h, np.array([0.0, 1.0])), [[1, 0], [3, 2], [5, 4]])
    y = P.causal_conv(h, np.array([[10.0, 1.0], [0.0, 2.0]]), np.array([0.5, 0.0]))
    assert np.allclose(y, [[1.5, 4], [3 + 10 + 0.5, 8], [5 + 30 + 0.5, 12]])       # the last column meets the current token


def test_the_plain_forget_gated_state_with_a_constant_gate():
    """With W_f = 0 the gate is a constant f per channel and o_t = sum_s f^(t-s) (1 - f) (q_t . 1) v_s."""
    D, d, dv, T = 4, 3, 2, 5
    rng = np.random.default_rng(0)
    W = {"q": rng.normal(size=(d, D)), "f": np.zeros((d, D)), "f.b": np.zeros(d), "lower": np.full(d, 0.5), "v": rng.normal(size=(dv, D)),
         "norm": np.ones(dv), "o": np.eye(dv)}
    h = rng.normal(size=(T, D))
    f = 0.5 + 0.5 * 0.5
    q, v = P.silu(h @ W["q"].T), h @ W["v"].T
    o = np.array([sum(f ** (t - s) * (1 - f) * q[t].sum() * v[s] for s in range(t + 1)) for t in range(T)])
    assert np.allclose(P.hgrn2(h, W, "", dict(heads=1, dim=d, vdim=dv), 1e-6), P.rms_norm(o, 1.0, 1e-6))


def test_the_plain_selective_scan_with_one_token():
    """One token from a zero state: y = dt x (B . C) + D x."""
    D, n, N, R = 3, 2, 4, 1
    rng = np.random.default_rng(1)
    W = {"in": rng.normal(size=(2 * n, D)), "conv": np.array([[0.0, 1.0]] * n), "conv.b": np.zeros(n), "x": rng.normal(size=(R + 2 * N, n)),
         "dt": rng.normal(size=(n, R)), "dt.b": rng.normal(size=n), "A_log": rng.normal(size=(n, N)), "D": rng.normal(size=n), "o": np.eye(n)}
    h = rng.normal(size=(1, D))
    xz = h @ W["in"].T
    x, z = P.silu(xz[:, :n]), xz[:, n:]
    low = x @ W["x"].T
    dt = P.softplus(low[:, :R] @ W["dt"].T + W["dt.b"])
    y = dt * x * (low[0, R:R + N] @ low[0, R + N:]) + W["D"] * x
    assert np.allclose(P.mamba1(h, W, "", dict(inner=n, state=N, dt_rank=R, conv=2)), y * P.silu(z))


def test_the_plain_router_picks_the_largest_and_the_lower_index_of_a_tie():
    D = 3
    W = {"router": np.zeros((4, D)), "router.b": np.array([1.0, 2.0, 2.0, 0.0])}
    for e in range(4):
        W.update({f"e{e}.gate": np.ones((1, D)), f"e{e}.up": np.ones((1, D)), f"e{e}.down": np.full((D, 1), 10.0 ** e)})
    h = np.ones((1, D))
    unit = P.silu(3.0) * 3.0
    mlp = dict(router=dict(experts=4, top=1), expert=dict(ff=1), shared=None)
    assert np.allclose(P.routed_experts(h, W, "", mlp), unit * 10.0)                       # expert 1, not 2
    mlp["router"]["top"] = 3
    w = np.exp([0.0, 0.0, -1.0])
    w /= w.sum()
    assert np.allclose(P.routed_experts(h, W, "", mlp), unit * (w[0] * 10 + w[1] * 100 + w[2] * 1))


def test_the_plain_latent_attention_sees_no_later_token_and_all_earlier_ones():
    cfg = zt.config(50, 16, [zt.layer(zt.latent(2, 4, 6, 8, 10, 0.5), None)])
    w = zt.make_weights(cfg, 3)
    a = zt.plain_logits(cfg, w, [1, 2, 3, 4, 5, 6])
    b = zt.plain_logits(cfg, w, [1, 2, 3, 4, 9, 6])
    c = zt.plain_logits(cfg, w, [7, 2, 3, 4, 5, 6])
    assert np.allclose(a[:4], b[:4]) and not np.allclose(a[5], b[5])
    assert not np.allclose(a[5], c[5], atol=1e-3)
