"""The kernels that Vavelorn brought, each alone against the plain functions (tests/plain_vavelorn.py):
layer norm, the sum between two norms, the gate on the second token table, interleaved rotation with the
cache write, chunked and softly capped attention (plain kernel, matrix-core prompt and decode kernels,
the fused decode kernel) with one sharp key just inside and just outside a chunk and at page borders,
the latent's norm and store, the per-head maps, a far key over the latent, the recurrence's inputs with
one decay per head, the silu-gated head norm."""

import numpy as np
import pytest
import torch

import plain_vavelorn as plain
from vavelorn_common import assert_close

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(array, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(array)).to(device=DEVICE, dtype=dtype)


def rounded(array, dtype):
    """The values a tensor of ``dtype`` holds of ``array``, in float64."""
    return torch.from_numpy(np.ascontiguousarray(array)).to(TORCH[dtype]).to(torch.float64).numpy()


# ----- norms --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("hidden", [40, 192, 1000, 4100])
def test_layer_norm_rows(hidden):
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(hidden)
    x = rng.normal(3.0, 2.0, size=(9, hidden))          # a mean that is large beside the spread
    w = rng.uniform(0.5, 1.5, hidden)
    want = plain.layer_norm(rounded(x, "float32"), w, 1e-5)
    got = ops.layernorm_rows(dev(x), dev(w), 1e-5, torch.float32).cpu().numpy()
    assert_close(got, want, "float32", f"layer norm {hidden}")
    index = [7, 0, 7, 3]
    got = ops.layernorm_rows(dev(x), dev(w), 1e-5, torch.bfloat16, row_index=dev(index, torch.int32)).float().cpu().numpy()
    assert_close(got, want[index], "bfloat16", f"layer norm {hidden}, gathered rows")


@pytest.mark.parametrize("hidden", [40, 1000, 5000])
@pytest.mark.parametrize("centered", [False, True])
def test_sum_between_two_norms(hidden, centered):
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(hidden + centered)
    x, a = rng.normal(1.0, 2.0, size=(5, hidden)), rng.normal(-0.5, 3.0, size=(5, hidden))
    w, w_next = rng.uniform(0.5, 1.5, hidden), rng.uniform(0.5, 1.5, hidden)
    eps, eps_next = 1e-5, 1e-6
    x32, a32 = rounded(x, "float32"), rounded(a, "float32")
    new_x = x32 + (plain.layer_norm(a32, w, eps) if centered else plain.rms(a32, eps) * w)
    readers = {ops.NEXT_NOTHING: None, ops.NEXT_ROUNDED: new_x, ops.NEXT_RMS: plain.rms(new_x, eps_next) * w_next,
               ops.NEXT_CENTERED: plain.layer_norm(new_x, w_next, eps_next)}
    for kind, want in readers.items():
        for dtype in ("float32", "bfloat16"):
            rows = dev(x)
            got = ops.norm_add_norm_(rows, dev(a), dev(w), centered, eps, next_kind=kind, next_weight=dev(w_next), next_eps=eps_next,
                                     next_dtype=TORCH[dtype])
            assert_close(rows.cpu().numpy(), new_x, "float32", f"new rows, kind {kind}")
            if want is None:
                assert got is None
            else:
                assert got.dtype == TORCH[dtype]
                assert_close(got.float().cpu().numpy(), want, dtype, f"what follows, kind {kind}")


def test_gate_on_the_token_table():
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(0)
    table = rounded(rng.normal(size=(50, 36)), "bfloat16")
    z = rounded(rng.normal(0.0, 2.0, size=(70, 12)), "float32")
    ids = rng.integers(0, 50, size=70)
    want = plain.gelu_tanh(z) * table[ids][:, 24:36]
    for dtype in ("float32", "bfloat16"):
        got = ops.gelu_gate_rows(dev(z), dev(table, TORCH[dtype]), dev(ids, torch.int32), 24, TORCH[dtype])
        assert_close(got.float().cpu().numpy(), want, dtype, "gated table rows")
    np.testing.assert_allclose(plain.gelu_tanh(np.array([0.0, 1.0, -1.0, 3.0])), [0.0, 0.841192, -0.158808, 2.996363], atol=1e-6)


# ----- attention: rotation, cache write, chunks, soft cap ---------------------------------------------------
class Sequence:
    """One sequence's raw projections written to a paged cache through the product's kernels, in portions."""

    def __init__(self, q, k, v, dtype, rot_dims, base, cuts, pages_order=None):
        from flyweight_amd.kernels import ops
        self.T, self.H, self.d = q.shape
        self.G, self.dv = k.shape[1], v.shape[2]
        self.dtype = dtype
        blocks = (self.T + 63) // 64
        order = list(pages_order) if pages_order is not None else list(range(blocks))[::-1]      # pages out of order
        self.k_pages = torch.full((blocks + 2, self.G, 64, self.d), 7.0, dtype=TORCH[dtype], device=DEVICE)     # stale values everywhere
        self.v_pages = torch.full((blocks + 2, self.G, self.dv, 64), -7.0, dtype=TORCH[dtype], device=DEVICE)
        self.table = dev(np.asarray(order, dtype=np.int32)[None, :], torch.int32)
        half = rot_dims // 2
        inv_freq = torch.tensor(base ** (-2.0 * np.arange(half) / max(rot_dims, 1)), dtype=torch.float64, device=DEVICE)
        qkv = np.concatenate([q.reshape(self.T, -1), k.reshape(self.T, -1), v.reshape(self.T, -1)], axis=1)
        self.queries, at = [], 0
        for n in cuts:
            n = min(n, self.T - at)
            pos = dev(np.arange(at, at + n), torch.int32)
            cos, sin = ops.rope_table(pos, inv_freq) if half else (None, None)
            seg = torch.zeros(n, dtype=torch.int32, device=DEVICE)
            self.queries.append(ops.qk_norm_rope_kv_write(dev(qkv[at:at + n]), self.H, self.G, self.d, None, None, 1.0, cos, sin, rot_dims,
                                                          self.k_pages, self.v_pages, self.table, seg, pos, v_dim=self.dv, interleaved=True))
            at += n
            if at >= self.T:
                break
        self.q = torch.cat(self.queries)


def sharp_inputs(T, H, G, d, dv, sharp_keys, rng, strength=4.5):
    """Random projections in which the keys at ``sharp_keys`` point along every query: whoever sees one of
    them gives it nearly all its weight, so a mask that is one key off changes the output visibly."""
    q = rng.normal(size=(T, H, d)) * 0.3
    k = rng.normal(size=(T, G, d)) * 0.3
    v = rng.normal(size=(T, G, dv))
    direction = rng.normal(size=d)
    direction /= np.linalg.norm(direction)
    q += strength * direction
    for j in sharp_keys:
        k[j] += strength * direction
    return q, k, v


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunk,rot_dims,d,dv,cap", [(64, 0, 32, 32, None), (65, 16, 32, 48, 30.0), (63, 32, 32, 16, 4.0),
                                                      (112, 20, 80, 96, 40.0), (1, 8, 16, 16, None), (None, 64, 64, 128, 8.0),
                                                      (40, 4, 20, 12, 5.0)])
def test_chunked_attention_with_a_sharp_key_at_every_edge(dtype, chunk, rot_dims, d, dv, cap):
    """Keys at the first and last place of every chunk are sharp: rows see the sharp first key of their own
    chunk and never the sharp last key of the chunk before. The whole sequence as a prompt in portions
    (cut inside chunks and pages), then every row once more as a decode step of its own."""
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(d + dv)
    T, H, G = 300, 4, 2
    size = chunk or T
    edges = sorted({j for j in range(T) if j % size in (0, size - 1)} | {63, 64, 128})
    q, k, v = sharp_inputs(T, H, G, d, dv, edges if chunk != 1 else [5], rng)
    q, k, v = (rounded(x, "float32") for x in (q, k, v))
    base, scale = 10000.0, 0.35
    positions = np.arange(T)
    want = plain.chunked_heads(plain.rotate_pairs(q, positions, rot_dims, base), plain.rotate_pairs(k, positions, rot_dims, base), v,
                               scale, chunk, cap).reshape(T, H * dv)
    cuts = [70, 2, 59, 64, 1, 33, 71]
    seq = Sequence(q, k, v, dtype, rot_dims, base, cuts)
    # a prompt in portions: every portion attends against what the earlier ones stored
    outs, at = [], 0
    for n, queries in zip(cuts, seq.queries):
        n = queries.shape[0]

        class Ctx:
            all_decode, decode_prefix, max_context = False, 0, at + n
            row_seg = torch.zeros(n, dtype=torch.int32, device=DEVICE)
            row_pos = dev(np.arange(at, at + n), torch.int32)
            seg_row0 = dev([0, n], torch.int32)
        tile_seg, tile_row0 = ops.query_tiles([0, n])
        outs.append(ops.attention(queries, H, G, d, seq.k_pages, seq.v_pages, seq.table, Ctx, scale, 0, tile_seg=dev(tile_seg, torch.int32),
                                  tile_row0=dev(tile_row0, torch.int32), v_dim=dv, chunk=chunk or 0, softcap=cap or 0.0))
        at += n
    assert_close(torch.cat(outs).float().cpu().numpy(), want, dtype, f"prompt in portions, chunk {chunk}", scale=1.0)
    # every row as a single-token step (a batch of 20 rows of one sequence each would need 20 caches: rows
    # of one sequence at different positions serve as well, the kernels take a position per row)
    rows = sorted(set(edges + [e + 1 for e in edges if e + 1 < T] + [T - 1, 1, 0]))
    picked = seq.q[rows]

    class Decode:
        all_decode, decode_prefix, max_context = True, 0, T
        row_seg = torch.zeros(len(rows), dtype=torch.int32, device=DEVICE)
        row_pos = dev(rows, torch.int32)
    got = ops.attention(picked, H, G, d, seq.k_pages, seq.v_pages, seq.table, Decode, scale, 0, v_dim=dv, chunk=chunk or 0, softcap=cap or 0.0)
    assert_close(got.float().cpu().numpy(), want[rows], dtype, f"single rows, chunk {chunk}", scale=1.0)


@pytest.mark.parametrize("chunk,rot_dims,d,dv,cap", [(65, 16, 32, 48, 30.0), (112, 20, 80, 96, 40.0), (None, 64, 64, 128, 8.0)])
def test_fused_decode_attention(chunk, rot_dims, d, dv, cap):
    """Rotation, cache write and attention of a single-token step in one kernel: the rows after a prompt,
    one by one, against the plain functions; what it stores serves the rows behind it."""
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(d)
    T, H, G, first = 200, 4, 2, 120
    size = chunk or T
    edges = [j for j in range(T) if j % size in (0, size - 1)] + [127, 128]
    q, k, v = sharp_inputs(T, H, G, d, dv, edges, rng)
    q, k, v = (rounded(x, "float32") for x in (q, k, v))
    base, scale = 5000.0, 0.3
    positions = np.arange(T)
    want = plain.chunked_heads(plain.rotate_pairs(q, positions, rot_dims, base), plain.rotate_pairs(k, positions, rot_dims, base), v,
                               scale, chunk, cap).reshape(T, H * dv)
    seq = Sequence(q[:first], k[:first], v[:first], "bfloat16", rot_dims, base, [first], pages_order=[3, 0, 2, 1])
    half = rot_dims // 2
    inv_freq = torch.tensor(base ** (-2.0 * np.arange(half) / max(rot_dims, 1)), dtype=torch.float64, device=DEVICE)
    qkv = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], axis=1)
    seg = torch.zeros(1, dtype=torch.int32, device=DEVICE)
    got = []
    for t in range(first, T):
        pos = dev([t], torch.int32)
        cos, sin = ops.rope_table(pos, inv_freq)
        got.append(ops.attention_decode_fused(dev(qkv[t:t + 1]), H, G, d, None, None, 1.0, cos, sin, rot_dims, seq.k_pages, seq.v_pages,
                                              seq.table, seg, pos, scale, T, v_dim=dv, chunk=chunk or 0, softcap=cap or 0.0, interleaved=True))
    assert_close(torch.cat(got).float().cpu().numpy(), want[first:], "bfloat16", f"fused decode, chunk {chunk}", scale=1.0)


# ----- the latent ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rank", [8, 40, 64, 128, 256, 320])
def test_latent_norm_and_store(dtype, rank):
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(rank)
    T = 150
    raw = rounded(rng.normal(0.0, 3.0, size=(T, rank + 9)), "float32")      # the latent's columns lie in wider rows
    w = rng.uniform(0.5, 1.5, rank)
    want = plain.rms(raw[:, :rank], 1e-5) * w
    k_pages = torch.zeros((4, 1, 64, rank), dtype=TORCH[dtype], device=DEVICE)
    v_pages = torch.zeros((4, 1, rank, 64), dtype=TORCH[dtype], device=DEVICE)
    table = dev([[2, 0, 3]], torch.int32)
    ops.latent_norm_write(dev(raw)[:, :rank], dev(w), 1e-5, k_pages, v_pages, table, torch.zeros(T, dtype=torch.int32, device=DEVICE),
                          dev(np.arange(T), torch.int32))
    order = [2, 0, 3]
    keys = torch.cat([k_pages[p, 0] for p in order]).float().cpu().numpy()[:T]
    values = torch.cat([v_pages[p, 0].T for p in order]).float().cpu().numpy()[:T]
    assert_close(keys, want, dtype, "latent as keys")
    assert np.array_equal(keys, values)
    assert float(k_pages[1].abs().max()) == 0.0         # the page of nobody stays as it was


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows,heads,n,k", [(1, 3, 40, 24), (70, 2, 64, 16), (130, 5, 9, 100), (64, 1, 128, 128)])
def test_map_per_head(dtype, rows, heads, n, k):
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(rows + n)
    x = rounded(rng.normal(size=(rows, heads * k + 5)), dtype)
    w = rounded(rng.normal(size=(heads, n, k)) / np.sqrt(k), dtype)
    gate = rounded(rng.normal(0.0, 2.0, size=(rows, 3 + heads * n)), "float32")
    plain_map = np.einsum("rhk,hnk->rhn", x[:, :heads * k].reshape(rows, heads, k), w).reshape(rows, heads * n)
    got = ops.head_linear(dev(x, TORCH[dtype])[:, :heads * k], dev(w, TORCH[dtype]), TORCH[dtype])
    assert_close(got.float().cpu().numpy(), plain_map, dtype, "map per head")
    got = ops.head_linear(dev(x, TORCH[dtype])[:, :heads * k], dev(w, TORCH[dtype]), TORCH[dtype], gate=dev(gate)[:, 3:])
    assert_close(got.float().cpu().numpy(), plain_map * plain.sigmoid(gate[:, 3:]), dtype, "gated map per head")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_over_the_latent(dtype):
    """Six heads over one shared latent head, 700 tokens: one token far back (and one just across a page
    border from it) carries a latent along the queries and takes nearly all the weight of every later row,
    in a prompt's tiles and in single-token steps."""
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(11)
    T, H, rank = 700, 6, 64
    c = rng.normal(size=(T, rank)) * 0.3
    q = rng.normal(size=(T, H, rank)) * 0.3
    direction = np.ones(rank) / np.sqrt(rank)
    q += 5.0 * direction
    for far in (63, 64):
        c[far] += 5.0 * direction
    c, q = rounded(c, dtype), rounded(q, dtype)
    k_pages = torch.zeros((12, 1, 64, rank), dtype=TORCH[dtype], device=DEVICE)
    v_pages = torch.zeros((12, 1, rank, 64), dtype=TORCH[dtype], device=DEVICE)
    table = dev([list(range(11))[::-1]], torch.int32)
    ones = np.ones(rank)
    # stored without a change: the norm's own scale is undone by the weight
    norm = np.sqrt(np.mean(c * c, axis=-1, keepdims=True) + 1e-12)
    ops.latent_norm_write(dev(c / norm * 1.0), dev(ones), 1e-12, k_pages, v_pages, table, torch.zeros(T, dtype=torch.int32, device=DEVICE),
                          dev(np.arange(T), torch.int32))
    c_stored = torch.cat([k_pages[p, 0] for p in range(10, -1, -1)]).float().cpu().numpy()[:T]
    want_unit = np.zeros((T, H, rank))
    for i in range(T):
        for head in range(H):
            want_unit[i, head] = plain.softmax_rows((c_stored[:i + 1].astype(np.float64) @ q[i, head]) * 0.4) @ c_stored[:i + 1]

    class Ctx:
        all_decode, decode_prefix, max_context = False, 0, T
        row_seg = torch.zeros(T, dtype=torch.int32, device=DEVICE)
        row_pos = dev(np.arange(T), torch.int32)
        seg_row0 = dev([0, T], torch.int32)
    tile_seg, tile_row0 = ops.query_tiles([0, T])
    queries = dev(q.reshape(T, H * rank), TORCH[dtype])
    got = ops.attention(queries, H, 1, rank, k_pages, v_pages, table, Ctx, 0.4, 0, tile_seg=dev(tile_seg, torch.int32),
                        tile_row0=dev(tile_row0, torch.int32), v_dim=rank)
    assert_close(got.float().cpu().numpy(), want_unit.reshape(T, H * rank), dtype, "prompt over the latent", scale=1.0)
    rows = [62, 63, 64, 65, 127, 128, 400, 699]

    class Decode:
        all_decode, decode_prefix, max_context = True, 0, T
        row_seg = torch.zeros(len(rows), dtype=torch.int32, device=DEVICE)
        row_pos = dev(rows, torch.int32)
    got = ops.attention(queries[rows].contiguous(), H, 1, rank, k_pages, v_pages, table, Decode, 0.4, 0, v_dim=rank)
    assert_close(got.float().cpu().numpy(), want_unit.reshape(T, H * rank)[rows], dtype, "single rows over the latent", scale=1.0)
    # the far keys hold the weight of the last row
    weights = plain.softmax_rows((c_stored.astype(np.float64) @ q[699, 0]) * 0.4)
    assert weights[63] + weights[64] > 0.9


# ----- the recurrence's inputs and its gated norm ---------------------------------------------------------------
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,taps", [(4, 2, 24, 40, 4), (3, 3, 40, 24, 2), (2, 1, 64, 64, 3), (1, 1, 4, 4, 1)])
def test_recurrence_inputs_with_one_decay_per_head(heads, kv_heads, dim, vdim, taps):
    """Two segments of unequal length that continue sequences (their convolution memory is given), then
    single-token steps that move the memory on: q, k, v, beta and the decays as the plain functions give
    them, the decay alike in every key channel of a head."""
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(heads * dim)
    D = 32
    p = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}
    channels = 2 * kv_heads * dim + heads * vdim
    w = {"q": rng.normal(size=(kv_heads * dim, D)) * 0.3, "k": rng.normal(size=(kv_heads * dim, D)) * 0.3,
         "v": rng.normal(size=(heads * vdim, D)) * 0.3, "b": rng.normal(size=(heads, D)) * 0.3, "a": rng.normal(size=(heads, D)) * 0.3,
         "q.conv": rng.normal(size=(kv_heads * dim, taps)) * 0.5, "k.conv": rng.normal(size=(kv_heads * dim, taps)) * 0.5,
         "v.conv": rng.normal(size=(heads * vdim, taps)) * 0.5, "A_log": rng.uniform(-3, 0.5, heads), "dt_bias": rng.uniform(-3, 0, heads)}
    lengths = [13, 5]
    h = [rng.normal(size=(n, D)) for n in lengths]
    before = [{n: rng.normal(size=(taps - 1, w[n].shape[0])) for n in "qkv"} for _ in lengths]
    state = torch.zeros((3, channels, taps - 1), dtype=torch.float32, device=DEVICE)
    slots = [2, 0]
    for slot, memory in zip(slots, before):
        state[slot] = dev(np.concatenate([memory[n] for n in "qkv"], axis=1).T)
    proj = np.concatenate([np.concatenate([x @ w[n].T for n in ("q", "k", "v", "b", "a")], axis=1) for x in h])
    rows = sum(lengths)
    taps_all = dev(np.concatenate([w["q.conv"], w["k.conv"], w["v.conv"]]))
    row_seg = dev(np.repeat([0, 1], lengths), torch.int32)
    seg_row0 = dev([0, lengths[0], rows], torch.int32)
    proj_dev = dev(proj)
    records = ops.delta_prepare(proj_dev, channels, proj_dev[:, channels + heads:channels + 2 * heads], taps_all, state, dev(w["A_log"]),
                                dev(w["dt_bias"]), row_seg, seg_row0, dev(slots, torch.int32), 2, heads, kv_heads, dim, vdim,
                                decay_per_head=True).cpu().numpy()
    d4, v4 = (dim + 3) // 4 * 4, (vdim + 3) // 4 * 4
    at = 0
    for segment, (x, memory) in enumerate(zip(h, before)):
        q, k, v, beta, decay, raw = plain.delta_inputs(x, w, p, memory)
        for head in range(heads):
            g = head // (heads // kv_heads)
            mine = records[at:at + len(x), head]
            assert_close(mine[:, :dim], q[:, g], "float32", "q")
            assert_close(mine[:, d4:d4 + dim], k[:, g], "float32", "k")
            assert_close(mine[:, 2 * d4:2 * d4 + dim], np.repeat(decay[:, head:head + 1], dim, axis=1), "float32", "decay")
            assert_close(mine[:, 3 * d4], beta[:, head], "float32", "beta")
            assert_close(mine[:, 3 * d4 + 4:3 * d4 + 4 + vdim], v[:, head], "float32", "v")
        if taps > 1:       # the memory moved on by the segment's rows
            joined = {n: np.concatenate([memory[n], raw[n]])[-(taps - 1):] for n in "qkv"}
            assert_close(state[slots[segment]].cpu().numpy(), np.concatenate([joined[n] for n in "qkv"], axis=1).T, "float32", "memory")
        at += len(x)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_norm_with_a_silu_gate(dtype):
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(5)
    rows, heads, vdim = 33, 3, 40
    o = rounded(rng.normal(0.0, 4.0, size=(rows, heads, vdim)), "float32")
    gate = rounded(rng.normal(0.0, 2.0, size=(rows, heads * vdim + 7)), "float32")
    w = rng.uniform(0.5, 1.5, vdim)
    want = (plain.rms(o, 1e-5) * w).reshape(rows, -1) * plain.silu(gate[:, 7:])
    got = ops.gated_head_norm(dev(o.reshape(rows, -1)), dev(gate)[:, 7:], dev(w), heads, vdim, 1e-5, TORCH[dtype], gate_silu=True)
    assert_close(got.float().cpu().numpy(), want, dtype, "silu-gated head norm")
