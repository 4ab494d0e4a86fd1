"""Vavelorn on the CPU: its configuration and tensor names, the cache entries it asks for, and the
plain model held against itself (a sequence in one piece against token by token with carried state, the
chunks' edges, the latent's two forms)."""

import copy

import numpy as np
import pytest

import plain_vavelorn as plain
from vavelorn_common import CONFIG_X, CONFIG_Y, CONFIG_Z, make_folder


def test_config_lowers_to_parts_and_names(tmp_path):
    from flyweight_amd.config import ConfigError, VavelornConfig, load_config
    from flyweight_amd.engine.model import declared_tensors
    for name, raw in (("X", CONFIG_X), ("Y", CONFIG_Y), ("Z", CONFIG_Z)):
        folder = str(tmp_path / name)
        make_folder(folder, raw)
        config = load_config(folder)                         # the model class by config.json
        assert isinstance(config, VavelornConfig)
        spec = config.model_spec()
        declared = declared_tensors(spec)
        assert {n: tuple(d.shape) for n, d in declared.items()} == plain.tensor_shapes(raw)
        assert config.to_dict() == raw
        assert [layer.mixer.kind for layer in config.layers] == [entry["type"] for entry in raw["layers"]]
        assert spec.lm_head_name == "head" and all(layer.arrangement == "sandwich_norm_residual" for layer in spec.layers)
    # what the keys lower to
    spec = VavelornConfig.from_dict(CONFIG_X).model_spec()
    first, last = spec.layers[0].mixer, spec.layers[3].mixer
    assert first.kind == "gqa_attention" and first["chunk"] == 40 and first["score_softcap"] == 3.0 and first["position"].kind == "rotary_interleaved"
    assert last["chunk"] is None and last["score_softcap"] is None and spec.layers[3].ffn is None
    assert spec.layers[2].mixer["decay"] == "head" and spec.layers[2].mixer["gate"] == "silu"
    assert spec.layers[1].params["token_input"]["first_column"] == 12 and spec.layers[1].params["token_input"]["table_columns"] == 48
    assert all("token_input" not in layer.params for layer in VavelornConfig.from_dict(CONFIG_Z).model_spec().layers)
    for path, value, match in ((("layers", 0, "type"), "serial", "type"), (("layers", 0, "mixer", "heads"), 3, "multiple"),
                               (("layers", 0, "mixer", "rot", "dims"), 34, "dims"), (("norm", "eps"), 0, "eps"),
                               (("layers", 0, "mlp", "kind"), "sparse", "kind"), (("layers", 1, "mixer", "kv_rank"), None, "kv_rank"),
                               (("layers", 2, "mixer", "conv"), 0, "conv"), (("token_side", "dim"), -1, "dim")):
        broken = copy.deepcopy(CONFIG_X)
        at = broken
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            VavelornConfig.from_dict(broken)


def test_cache_entries(tmp_path):
    """Attention layers ask for paged keys and values (one page group per distinct shape), a latent layer
    for one shared head of the latent's size, a recurrence for a matrix state and the convolutions' memory
    in the request's slot; slots and pages come back."""
    from flyweight_amd.cache import CacheManager
    from flyweight_amd.config import VavelornConfig
    from flyweight_amd.engine.model import CausalLM
    model = CausalLM(VavelornConfig.from_dict(CONFIG_X).model_spec())
    needs = model.cache_needs()
    assert needs[0].num_kv_heads == 2 and needs[0].head_dim == 32 and needs[0].v_head_dim == 48
    assert needs[1].num_kv_heads == 1 and needs[1].head_dim == 40
    assert set(needs[2]) == {"state", "conv"} and needs[2]["state"].shape == (4, 40, 24) and needs[2]["conv"].shape == (2 * 2 * 24 + 4 * 40, 3)
    cache = CacheManager(needs, num_pages=6, max_requests=2)
    assert len(cache.groups) == 3
    cache.admit("a")
    cache.reserve("a", 300)
    cache.commit("a", 300)
    # the chunked group (chunks of 40) keeps the pages from the chunk of the next token on: position 300 lies in
    # the chunk from 280, which begins in the fifth page; the groups that keep every key hold all five
    held = {g.need.chunk: g.pool.in_use for g in cache.groups}
    assert held == {40: 1, None: 5} and cache.groups[0].tables["a"][:4] == [-1, -1, -1, -1]
    cache.reserve("a", 321)
    cache.commit("a", 319)              # still in the chunk from 280: nothing more goes back
    assert cache.groups[0].pool.in_use == 2
    cache.commit("a", 320)              # the next token begins the chunk from 320, which lies in the sixth page
    assert cache.groups[0].pool.in_use == 1 and cache.groups[0].tables["a"][4] == -1
    cache.release("a")
    cache.check_invariants()
    assert all(g.pool.in_use == 0 for g in cache.groups)
    one_tap = CausalLM(VavelornConfig.from_dict(CONFIG_Z).model_spec()).cache_needs()
    assert set(one_tap[1]) == {"state"}         # one tap: no convolution memory


def _weights_of(config, layer, rng, scale=0.3):
    prefix = f"l{layer}.mix."
    shapes = {n[len(prefix):]: s for n, s in plain.tensor_shapes(config).items() if n.startswith(prefix)}
    return {n: rng.normal(size=s) * (scale if len(s) == 2 else 1.0) for n, s in shapes.items()}


def test_plain_recurrence_in_one_piece_and_token_by_token():
    rng = np.random.default_rng(0)
    p = CONFIG_X["layers"][2]["mixer"]
    w = _weights_of(CONFIG_X, 2, rng)
    h = rng.normal(size=(23, CONFIG_X["width"]))
    H, G, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q, k, v, beta, decay, _ = plain.delta_inputs(h, w, p)
    S = np.zeros((H, d, dv))
    before = {n: np.zeros((p["conv"] - 1, w[n].shape[0])) for n in "qkv"}
    for t in range(23):
        q1, k1, v1, beta1, decay1, raw = plain.delta_inputs(h[t:t + 1], w, p, before)
        for x, y in ((q1, q[t:t + 1]), (k1, k[t:t + 1]), (v1, v[t:t + 1]), (beta1, beta[t:t + 1]), (decay1, decay[t:t + 1])):
            np.testing.assert_allclose(x, y, atol=1e-12)
        before = {n: np.concatenate([before[n], raw[n]])[-(p["conv"] - 1):] for n in "qkv"}
    assert decay.shape == (23, H) and np.all((decay > 0) & (decay < 1))
    # the read-out sees the token's own write: with beta = 1, no decay and a unit key, o = v (k . q)
    S0, o = plain.delta_step(np.zeros((d, dv)), 2.0 * np.eye(d)[0], np.eye(d)[0], np.arange(dv, dtype=float), 1.0, 1.0)
    np.testing.assert_allclose(o, 2.0 * np.arange(dv))


def test_plain_chunks_and_rotation():
    """A row's output does not change with a key just outside its chunk and does with the chunk's first
    key; the rotation turns pairs of neighbours and leaves the channels past ``dims``."""
    rng = np.random.default_rng(1)
    p = CONFIG_X["layers"][0]["mixer"]
    w = _weights_of(CONFIG_X, 0, rng, scale=1.0)
    size = p["mask"]["size"]
    h = rng.normal(size=(size + 7, CONFIG_X["width"]))
    base = plain.chunked_attention(h, w, p)
    for moved_row, changes in ((size - 1, False), (size, True)):
        moved = h.copy()
        moved[moved_row] += 1.0
        assert (np.abs(plain.chunked_attention(moved, w, p)[size + 6] - base[size + 6]).max() > 1e-9) == changes
    x = rng.normal(size=(5, 2, 8))
    turned = plain.rotate_pairs(x, np.arange(5), 4, 100.0)
    np.testing.assert_array_equal(turned[..., 4:], x[..., 4:])
    np.testing.assert_array_equal(turned[0], x[0])
    angle = 3 * 100.0 ** (-2.0 / 4)
    np.testing.assert_allclose(turned[3, 1, 2:4], [x[3, 1, 2] * np.cos(angle) - x[3, 1, 3] * np.sin(angle),
                                                   x[3, 1, 3] * np.cos(angle) + x[3, 1, 2] * np.sin(angle)])
    np.testing.assert_allclose(np.sum(turned ** 2, axis=-1), np.sum(x ** 2, axis=-1))


def test_plain_latent_by_its_latent_alone():
    """Scores and outputs formed on the latent's side (the keys' map applied to the query, the values' map
    to the weighted latents) are those of the unfolded keys and values: only the latent has to be kept."""
    rng = np.random.default_rng(2)
    p = CONFIG_X["layers"][1]["mixer"]
    w = _weights_of(CONFIG_X, 1, rng, scale=0.5)
    eps = 1e-6
    h = rng.normal(size=(17, CONFIG_X["width"]))
    H, d, dv, rk = p["heads"], p["dim"], p["vdim"], p["kv_rank"]
    c = plain.rms(h @ w["dkv"].T, eps) * w["dkv.norm"]
    q = ((plain.rms(h @ w["dq"].T, eps) * w["dq.norm"]) @ w["uq"].T).reshape(17, H, d)
    out = np.zeros((17, H, dv))
    for head in range(H):
        q_latent = q[:, head] @ w["uk"].reshape(H, d, rk)[head]
        for i in range(17):
            mixed = plain.softmax_rows((c[:i + 1] @ q_latent[i]) * p["scale"]) @ c[:i + 1]
            out[i, head] = w["uv"].reshape(H, dv, rk)[head] @ mixed
    by_latent = (out.reshape(17, H * dv) * plain.sigmoid(h @ w["g"].T)) @ w["o"].T
    np.testing.assert_allclose(by_latent, plain.latent_attention(h, w, p, eps), atol=1e-10)


def test_plain_model_is_causal_and_every_part_counts():
    config = CONFIG_Y
    weights = plain.random_weights(config, 3)
    tokens = np.random.default_rng(4).integers(0, config["vocab"], size=50).tolist()
    layers = []
    whole = plain.forward(config, weights, tokens, layers)
    np.testing.assert_allclose(plain.forward(config, weights, tokens[:31]), whole[:31], atol=1e-9)
    assert len(layers) == len(config["layers"])
    for name in ("l0.mix.o", "l1.mix.o", "l2.mix.o", "l1.mlp.down", "l2.side.proj", "side.embed", "l3.norm1b", "l0.norm2b"):
        changed = dict(weights)
        # (a factor on a matrix in front of a norm would change nothing: its rows are turned round instead)
        changed[name] = weights[name][::-1].copy() if weights[name].ndim == 2 else weights[name] * np.linspace(0.5, 1.5, weights[name].size)
        assert np.abs(plain.forward(config, changed, tokens) - whole).max() > 1e-3, name
