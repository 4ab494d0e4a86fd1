"""Koketar on the CPU: its configuration and tensor names, the cache entries it asks for, and the
plain model held against itself (a sequence in one piece against token by token with carried state)."""

import copy

import numpy as np
import pytest

import plain_koketar as plain
from koketar_common import CONFIG_X, CONFIG_Y, file_config, make_folder


def test_config_lowers_to_parts_and_names(tmp_path):
    from flyweight_amd.config import ConfigError, KoketarConfig, load_config
    from flyweight_amd.engine.model import declared_tensors
    for name, raw in (("X", CONFIG_X), ("Y", CONFIG_Y)):
        folder = str(tmp_path / name)
        make_folder(folder, raw)
        config = load_config(folder)                         # the model class by config.json, the ranks by the tensors' shapes
        assert isinstance(config, KoketarConfig)
        assert [layer.right.decay_rank for layer in config.layers] == [l["mixer"]["right"]["rank_a"] for l in raw["layers"]]
        spec = config.model_spec()
        declared = declared_tensors(spec)
        assert {n: tuple(d.shape) for n, d in declared.items()} == plain.tensor_shapes(raw)
        assert spec.logit_softcap == raw.get("logit_softcap", 0.0)
        assert config.to_dict()["layers"][0]["mixer"]["left"]["rot"] == raw["layers"][0]["mixer"]["left"]["rot"]
    with pytest.raises(ConfigError, match="low-rank"):
        KoketarConfig.from_dict(file_config(CONFIG_X)).model_spec()     # without a checkpoint the ranks must be given
    for path, value, match in ((("layers", 0, "type"), "serial", "type"), (("layers", 1, "mixer", "left", "heads"), 3, "multiple"),
                               (("layers", 0, "mixer", "left", "rot", "dims"), 34, "dims"), (("norm", "eps"), 0, "eps"),
                               (("layers", 0, "mlp", "kind"), "sparse", "kind")):
        broken = copy.deepcopy(file_config(CONFIG_X))
        at = broken
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            KoketarConfig.from_dict(broken)


def test_cache_entries_of_a_layer_with_two_branches(tmp_path):
    """A layer's mixer asks for a mapping of needs: the windowed keys and values of the left branch
    (one page group per distinct shape and window), the matrix state and the convolutions' memory of
    the right one (slots). Pages the window has passed come back; slots are cleared when handed out."""
    from flyweight_amd.cache import CacheManager
    from flyweight_amd.config import load_config
    from flyweight_amd.engine.model import CausalLM
    folder = str(tmp_path / "X")
    make_folder(folder, CONFIG_X)
    model = CausalLM(load_config(folder).model_spec())
    needs = model.cache_needs()
    assert set(needs[0]) == {"left", "right"} and set(needs[0]["right"]) == {"state", "conv"}
    cache = CacheManager(needs, num_pages=6, max_requests=2)
    assert len(cache.groups) == 3 and sorted(g.need.window for g in cache.groups) == [5, 40, 70]
    assert (0, "left") in cache.needs and (1, "right", "state") in cache.needs
    assert cache.needs[(0, "left")].v_head_dim == 48 and cache.needs[(1, "left")].v_head_dim is None
    assert cache.needs[(1, "right", "state")].shape == (2, 80, 64) and cache.needs[(2, "right", "conv")].shape == (48, 3)
    cache.admit("a")
    cache.reserve("a", 300)
    cache.commit("a", 300)
    held = {g.need.window: g.pool.in_use for g in cache.groups}
    assert held[5] == 1 and held[40] == 1 and held[70] == 2          # only what the windows still see
    cache.release("a")
    cache.check_invariants()
    assert all(g.pool.in_use == 0 for g in cache.groups)


def test_plain_model_in_one_piece_and_token_by_token():
    """The oracle against itself: the recurrence over a whole sequence equals single steps that carry
    S and the convolutions' last inputs; the window keeps exactly ``size`` keys."""
    rng = np.random.default_rng(0)
    p = CONFIG_X["layers"][0]["mixer"]["right"]
    shapes = {n[len("l0.mix.right."):]: s for n, s in plain.tensor_shapes(CONFIG_X).items() if n.startswith("l0.mix.right.")}
    w = {n: rng.normal(size=s) * (0.3 if len(s) == 2 else 1.0) for n, s in shapes.items()}
    h = rng.normal(size=(23, CONFIG_X["width"]))
    whole = plain.gated_delta_rule(h, w, p, 1e-6)
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    S = np.zeros((H, d, dv))
    before = {n: np.zeros((p["conv"] - 1, w[n].shape[0])) for n in "qkv"}
    for t in range(23):
        q, k, v, beta, g, raw = plain.delta_inputs(h[t:t + 1], w, p, before)
        o = np.zeros((1, H, dv))
        for head in range(H):
            S[head], o[0, head] = plain.delta_rule_step(S[head], q[0, head // (H // G)], k[0, head // (H // G)], v[0, head], beta[0, head], g[0, head])
        np.testing.assert_allclose(plain.delta_output(o, h[t:t + 1], w, p, 1e-6)[0], whole[t], atol=1e-12)
        before = {n: np.concatenate([before[n], raw[n]])[-(p["conv"] - 1):] for n in "qkv"}
    # the window: a row's output does not change with a key `size` tokens back, and does with one `size - 1` back
    a = CONFIG_X["layers"][2]["mixer"]["left"]
    shapes = {n[len("l2.mix.left."):]: s for n, s in plain.tensor_shapes(CONFIG_X).items() if n.startswith("l2.mix.left.")}
    w = {n: rng.normal(size=s) for n, s in shapes.items()}
    h = rng.normal(size=(12, CONFIG_X["width"]))
    base = plain.window_attention(h, w, a, 1e-6)[11]
    size = a["mask"]["size"]
    for back, changes in ((size, False), (size - 1, True)):
        moved = h.copy()
        moved[11 - back] += 1.0
        assert (np.abs(plain.window_attention(moved, w, a, 1e-6)[11] - base).max() > 1e-9) == changes
