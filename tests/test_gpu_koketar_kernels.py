"""The kernels that Koketar brought, each alone against the plain functions of
tests/plain_koketar.py (float64), at sizes that are no multiple of anything: the recurrence over
segments with carried state, what the recurrence reads (convolutions with their memory, unit vectors,
decays), the gated head norm, the output norm that joins the residual stream, the clamped gated unit,
and attention whose values have a size of their own."""

import numpy as np
import pytest
import torch

import plain_koketar as plain

pytestmark = pytest.mark.gpu


def dev(array, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(array)).to(dtype).cuda()


def ints(values):
    return torch.tensor(list(values), dtype=torch.int32, device="cuda")


def record_layout(dim, vdim):
    """Where q, k, g, beta and v lie in what a token brings to a head: each of q, k, g and v rounded up
    to a multiple of four floats, beta and three unused floats in front of v."""
    d4, v4 = (dim + 3) // 4 * 4, (vdim + 3) // 4 * 4
    return {"q": 0, "k": d4, "g": 2 * d4, "beta": 3 * d4, "v": 3 * d4 + 4, "floats": 3 * d4 + 4 + v4}


@pytest.mark.parametrize("lengths,slots_of", [([37, 1, 18], [2, 0, 3]), ([150], [4]), ([70, 90], [1, 0])])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(3, 1, 20, 70), (2, 2, 64, 64), (4, 2, 8, 5), (1, 1, 130, 129), (2, 1, 256, 16)])
def test_recurrence_over_segments_with_carried_state(heads, kv_heads, dim, vdim, lengths, slots_of):
    """Short segments and single rows (a column of the state over sixteen lanes) and long ones of one or
    two sequences (over a whole wave), each from a state that is not zero."""
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(dim + vdim)
    rows = sum(lengths)
    q = plain.unit(rng.normal(size=(rows, kv_heads, dim))) * dim ** -0.5
    k = plain.unit(rng.normal(size=(rows, kv_heads, dim)))
    v = rng.normal(size=(rows, heads, vdim))
    beta = rng.uniform(0.1, 1.0, size=(rows, heads))
    decay = rng.uniform(0.5, 1.0, size=(rows, heads, dim))
    decay[:, 0, ::2] = 1.0                                      # channels that never forget
    start = rng.normal(size=(5, heads, dim, vdim))              # five slots, S[slot, head] as the equations write it
    state = dev(start.transpose(0, 1, 3, 2))                    # stored transposed
    at = record_layout(dim, vdim)
    assert at["floats"] == ops.delta_record_floats(dim, vdim)
    records = np.zeros((rows, heads, at["floats"]))
    for head in range(heads):
        g = head // (heads // kv_heads)
        records[:, head, at["q"]:at["q"] + dim] = q[:, g]
        records[:, head, at["k"]:at["k"] + dim] = k[:, g]
        records[:, head, at["g"]:at["g"] + dim] = decay[:, head]
        records[:, head, at["beta"]] = beta[:, head]
        records[:, head, at["v"]:at["v"] + vdim] = v[:, head]
    seg_row0 = np.concatenate([[0], np.cumsum(lengths)])
    out = ops.gated_delta_rule(dev(records), state, ints(seg_row0), ints(slots_of), len(lengths), heads, dim,
                               vdim).cpu().numpy().reshape(rows, heads, vdim)
    after = state.cpu().numpy().transpose(0, 1, 3, 2)
    for seg, (length, slot) in enumerate(zip(lengths, slots_of)):
        for head in range(heads):
            S = start[slot, head].copy()
            g = head // (heads // kv_heads)
            for t in range(seg_row0[seg], seg_row0[seg] + length):
                S, o = plain.delta_rule_step(S, q[t, g], k[t, g], v[t, head], beta[t, head], decay[t, head])
                np.testing.assert_allclose(out[t, head], o, rtol=0, atol=2e-5 * max(1.0, np.abs(o).max()))
            np.testing.assert_allclose(after[slot, head], S, rtol=0, atol=2e-5 * max(1.0, np.abs(S).max()))
    for slot in set(range(5)) - set(slots_of):                   # nobody's slots stay as they were
        np.testing.assert_array_equal(after[slot], start[slot].astype(np.float32))


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_what_the_recurrence_reads(taps):
    """Portions of one and of several rows behind a memory that is not zero: the convolutions see
    the inputs of the rows before the portion, then the memory holds the last taps - 1 inputs."""
    from flyweight_amd.kernels import ops
    heads, kv_heads, dim, vdim = 3, 1, 20, 70
    rng = np.random.default_rng(taps)
    channels = 2 * kv_heads * dim + heads * vdim
    lengths, slots_of = [5, 1, 2, 9], [1, 3, 0, 2]
    rows = sum(lengths)
    extra = 11                                                   # other columns ride in the same projection
    proj = rng.normal(size=(rows, channels + heads + extra))
    a = rng.normal(size=(rows, heads * dim)) * 2
    w = {"q.conv": rng.normal(size=(kv_heads * dim, taps)), "k.conv": rng.normal(size=(kv_heads * dim, taps)),
         "v.conv": rng.normal(size=(heads * vdim, taps))}
    A_log, dt_bias = rng.uniform(-2, 1, heads), rng.normal(size=heads * dim)
    memory = rng.normal(size=(4, channels, taps - 1))
    conv_state = dev(memory)
    seg_row0 = np.concatenate([[0], np.cumsum(lengths)])
    row_seg = np.repeat(np.arange(len(lengths)), lengths)
    wide = dev(np.concatenate([a, rng.normal(size=(rows, 5))], axis=1))      # the arguments as a view of wider rows
    records = ops.delta_prepare(dev(proj), channels, wide[:, :heads * dim], dev(np.concatenate([w["q.conv"], w["k.conv"], w["v.conv"]])),
                                conv_state, dev(A_log), dev(dt_bias), ints(row_seg), ints(seg_row0), ints(slots_of),
                                len(lengths), heads, kv_heads, dim, vdim).cpu().numpy()
    at = record_layout(dim, vdim)
    after = conv_state.cpu().numpy()
    # every head's record holds the q and k of its group (one group here), its own v, decays and strength
    for head in range(1, heads):
        np.testing.assert_array_equal(records[:, head, :at["g"]], records[:, 0, :at["g"]])
    assert (records[:, :, at["q"] + dim:at["k"]] == 0).all() and (records[:, :, at["v"] + vdim:] == 0).all()
    qkv = np.concatenate([records[:, 0, at["q"]:at["q"] + dim], records[:, 0, at["k"]:at["k"] + dim],
                          records[:, :, at["v"]:at["v"] + vdim].reshape(rows, -1)], axis=1)
    decay = records[:, :, at["g"]:at["g"] + dim].reshape(rows, -1)
    beta = records[:, :, at["beta"]]
    taps_all = np.concatenate([w["q.conv"], w["k.conv"], w["v.conv"]])
    for seg, (length, slot) in enumerate(zip(lengths, slots_of)):
        r0 = seg_row0[seg]
        x = proj[r0:r0 + length, :channels]
        before = memory[slot].T                                   # [taps - 1, channels]
        y = plain.silu(plain.causal_conv(x, taps_all, before))
        nq = kv_heads * dim
        want_q = plain.unit(y[:, :nq].reshape(length, kv_heads, dim)) * dim ** -0.5
        want_k = plain.unit(y[:, nq:2 * nq].reshape(length, kv_heads, dim))
        np.testing.assert_allclose(qkv[r0:r0 + length, :nq], want_q.reshape(length, -1), atol=3e-6, rtol=1e-5)
        np.testing.assert_allclose(qkv[r0:r0 + length, nq:2 * nq], want_k.reshape(length, -1), atol=3e-6, rtol=1e-5)
        np.testing.assert_allclose(qkv[r0:r0 + length, 2 * nq:], y[:, 2 * nq:], atol=1e-5, rtol=1e-5)
        want_g = np.exp(-np.exp(A_log)[None, :, None] * plain.softplus((a[r0:r0 + length] + dt_bias).reshape(length, heads, dim)))
        np.testing.assert_allclose(decay[r0:r0 + length], want_g.reshape(length, -1), atol=1e-6, rtol=1e-5)
        np.testing.assert_allclose(beta[r0:r0 + length], plain.sigmoid(proj[r0:r0 + length, channels:channels + heads]), atol=1e-6)
        if taps > 1:
            np.testing.assert_allclose(after[slot], np.concatenate([before, x])[-(taps - 1):].T, atol=1e-6)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gated_head_norm(out_dtype):
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(0)
    rows, heads, vdim, eps = 7, 3, 70, 1e-5
    o, gate, weight = rng.normal(size=(rows, heads, vdim)) * 3, rng.normal(size=(rows, heads, vdim)), rng.uniform(0.5, 1.5, vdim)
    got = ops.gated_head_norm(dev(o.reshape(rows, -1)), dev(gate.reshape(rows, -1)), dev(weight), heads, vdim, eps, out_dtype)
    want = (plain.rms(o, eps) * weight * plain.sigmoid(gate)).reshape(rows, -1)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, atol=1e-5 if out_dtype == torch.float32 else 2e-2, rtol=1e-5 if out_dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("hidden", [96, 1000, 5000])
@pytest.mark.parametrize("two", [False, True])
def test_output_norm_joins_the_residual_stream(hidden, two):
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(hidden)
    rows, eps, mult = 5, 1e-6, 0.3
    x, a, b, w = rng.normal(size=(rows, hidden)), rng.normal(size=(rows, hidden)), rng.normal(size=(rows, hidden)), rng.uniform(-0.3, 0.3, hidden)
    y = 0.8 * a + (0.5 * b if two else 0.0)
    want = x + mult * plain.output_norm(y, w, eps)
    xd = dev(x)
    rounded = ops.norm_scale_add_(xd, dev(a), dev(w), eps, mult, b=dev(b) if two else None, scale_a=0.8, scale_b=0.5,
                                  one_centered=True, rounded_dtype=torch.bfloat16)
    np.testing.assert_allclose(xd.cpu().numpy(), want, atol=2e-6, rtol=1e-5)
    assert torch.equal(rounded, xd.to(torch.bfloat16))


def test_clamped_gated_unit():
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(1)
    rows, inter, limit = 6, 75, 0.7
    gate_up = rng.normal(size=(rows, 2 * inter)) * 2
    gate, up = np.minimum(gate_up[:, :inter], limit), np.clip(gate_up[:, inter:], -limit, limit)
    want = gate * plain.sigmoid(1.702 * gate) * (up + 1.0)
    got = ops.clamped_glu(dev(gate_up), limit, 1.702, 1.0, torch.float32)
    np.testing.assert_allclose(got.cpu().numpy(), want, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_with_values_of_their_own_size(dtype):
    """One sharp key per row: the query of row i is made to match the key `back[i]` tokens before it,
    which lies just inside the window, just outside it (the row then falls back on the rest), at a
    page's border or far back. Values are wider than keys."""
    from flyweight_amd.kernels import ops
    torch_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(2)
    heads, kv_heads, dim, vdim, window, scale = 2, 1, 16, 40, 70, 1.0
    rows = 200
    k = plain.unit(rng.normal(size=(rows, kv_heads, dim))) * 4.0
    v = rng.normal(size=(rows, kv_heads, vdim))
    back = rng.choice([0, 1, 5, 63, 64, 65, window - 2, window - 1, window, window + 1], size=rows)
    q = np.stack([np.stack([k[max(0, i - back[i]), 0] * 2.0] * heads) for i in range(rows)])
    qkv = np.concatenate([q.reshape(rows, -1), k.reshape(rows, -1), v.reshape(rows, -1)], axis=1)
    pages = 5
    k_pages = torch.zeros((pages, kv_heads, 64, dim), dtype=torch_dtype, device="cuda")
    v_pages = torch.zeros((pages, kv_heads, vdim, 64), dtype=torch_dtype, device="cuda")
    table = ints([3, 0, 4, 1]).view(1, 4)
    row_seg, row_pos = ints([0] * rows), ints(range(rows))
    q_out = ops.qk_norm_rope_kv_write(dev(qkv), heads, kv_heads, dim, None, None, 1.0, None, None, 0, k_pages, v_pages, table,
                                      row_seg, row_pos, v_dim=vdim)
    got = ops.attention_generic(q_out, heads, kv_heads, dim, k_pages, v_pages, table, row_seg, row_pos, scale, window, v_dim=vdim)
    got = got.float().cpu().numpy().reshape(rows, heads, vdim)
    if dtype == "bfloat16":     # what the cache holds
        q, k, v = (torch.from_numpy(t).to(torch.bfloat16).double().numpy() for t in (q, k, v))
    for i in range(rows):
        lo = max(0, i - window + 1)
        for head in range(heads):
            score = (k[lo:i + 1, 0] @ q[i, head]) * scale
            weight = np.exp(score - score.max())
            want = (weight / weight.sum()) @ v[lo:i + 1, 0]
            np.testing.assert_allclose(got[i, head], want, atol=1e-4 if dtype == "float32" else 3e-2, err_msg=f"row {i} back {back[i]}")


@pytest.mark.parametrize("head_dim,v_dim", [(16, 48), (64, 128), (128, 64), (48, 16), (32, 32)])
@pytest.mark.parametrize("window", [0, 70])
def test_matrix_core_attention_with_values_of_their_own_size(head_dim, v_dim, window):
    """The tiled prompt kernel, the split-key decode kernel and the decode kernel that norms, rotates
    and stores on its way, against the generic kernel on the same pages (bfloat16): keys and values of
    different sizes, queries made to match single keys near the window's edge and at page borders."""
    from flyweight_amd.kernels import ops
    rng = np.random.default_rng(head_dim * 7 + v_dim)
    heads, kv_heads, scale, rows = 4, 2, 0.7, 200
    k = plain.unit(rng.normal(size=(rows + 1, kv_heads, head_dim))) * 3.0
    v = rng.normal(size=(rows + 1, kv_heads, v_dim))
    back = rng.choice([0, 1, 63, 64, 65, 68, 69, 70, 71], size=rows + 1)
    q = np.stack([np.stack([k[max(0, i - back[i]), h // 2] * 2.0 for h in range(heads)]) for i in range(rows + 1)])
    qkv = np.concatenate([q.reshape(rows + 1, -1), k.reshape(rows + 1, -1), v.reshape(rows + 1, -1)], axis=1)
    pages = 6
    k_pages = torch.zeros((pages, kv_heads, 64, head_dim), dtype=torch.bfloat16, device="cuda")
    v_pages = torch.zeros((pages, kv_heads, v_dim, 64), dtype=torch.bfloat16, device="cuda")
    v_pages.fill_(9.0)          # what an earlier owner left behind the sequence's end must not count
    table = ints([5, 0, 3, 1]).view(1, 4)
    row_seg, row_pos = ints([0] * rows), ints(range(rows))
    q_rows = ops.qk_norm_rope_kv_write(dev(qkv[:rows]), heads, kv_heads, head_dim, None, None, 1.0, None, None, 0, k_pages, v_pages,
                                       table, row_seg, row_pos, v_dim=v_dim)
    want = ops.attention_generic(q_rows, heads, kv_heads, head_dim, k_pages, v_pages, table, row_seg, row_pos, scale, window, v_dim=v_dim)
    tile_seg, tile_row0 = ops.query_tiles([0, rows])
    got = ops.attention_prefill(q_rows, heads, kv_heads, head_dim, k_pages, v_pages, table, ints(tile_seg), ints(tile_row0),
                                ints([0, rows]), row_pos, scale, window, v_dim=v_dim)
    assert got.shape == (rows, heads * v_dim)
    np.testing.assert_allclose(got.float().cpu().numpy(), want.float().cpu().numpy(), atol=4e-2, rtol=2e-2)
    # one row per request: the rows at positions 130 and 199 of the same sequence, as two requests on the same pages
    two = ints([130, 199])
    both_tables = table.repeat(2, 1).contiguous()
    got = ops.attention_decode(q_rows[[130, 199]].contiguous(), heads, kv_heads, head_dim, k_pages, v_pages, both_tables, ints([0, 1]), two,
                               scale, 256, window, v_dim=v_dim)
    np.testing.assert_allclose(got.float().cpu().numpy(), want[[130, 199]].float().cpu().numpy(), atol=4e-2, rtol=2e-2)
    # the next token from its raw projections: stored and attended in one kernel, against the two kernels on a copy
    k_copy, v_copy = k_pages.clone(), v_pages.clone()
    last = dev(qkv[rows:rows + 1])
    q_last = ops.qk_norm_rope_kv_write(last, heads, kv_heads, head_dim, None, None, 1.0, None, None, 0, k_copy, v_copy, table,
                                       ints([0]), ints([rows]), v_dim=v_dim)
    want_last = ops.attention_generic(q_last, heads, kv_heads, head_dim, k_copy, v_copy, table, ints([0]), ints([rows]), scale, window, v_dim=v_dim)
    got_last = ops.attention_decode_fused(last, heads, kv_heads, head_dim, None, None, 1.0, None, None, 0, k_pages, v_pages, table,
                                          ints([0]), ints([rows]), scale, 256, window, v_dim=v_dim)
    np.testing.assert_allclose(got_last.float().cpu().numpy(), want_last.float().cpu().numpy(), atol=4e-2, rtol=2e-2)
    assert torch.equal(k_pages, k_copy) and torch.equal(v_pages, v_copy)


@pytest.mark.parametrize("rows", [1, 8, 16, 40, 64, 200])
def test_clamped_gated_unit_behind_its_product(rows):
    """Few rows: the unit is the epilogue of the gate|up product (the decode product up to 16 rows, the
    split-K product up to 64); more rows: float32 sums and the unit's own kernel. All against the plain formula."""
    from flyweight_amd.parts.linear import Linear
    rng = np.random.default_rng(rows)
    hidden, inter, limit = 320, 448, 0.9
    a = torch.from_numpy(rng.normal(size=(rows, hidden))).to(torch.bfloat16).cuda()
    w = torch.from_numpy(rng.normal(size=(2 * inter, hidden)) / 8).to(torch.bfloat16).cuda()
    got = Linear(w).clamped_glu(a, limit, 1.702, 1.0).float().cpu().numpy()
    sums = a.double().cpu().numpy() @ w.double().cpu().numpy().T
    gate, up = np.minimum(sums[:, :inter], limit), np.clip(sums[:, inter:], -limit, limit)
    want = gate * plain.sigmoid(1.702 * gate) * (up + 1.0)
    np.testing.assert_allclose(got, want, atol=1.5e-2, rtol=1e-2)
    # the plain unit through the same products is what it was: silu(gate) * up
    plain_unit = Linear(w).swiglu(a).float().cpu().numpy()
    np.testing.assert_allclose(plain_unit, plain.silu(sums[:, :inter]) * sums[:, inter:], atol=3e-2, rtol=1.5e-2)
