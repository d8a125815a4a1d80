"""The Sonodra architecture against the plain implementation of tests/plain_sonodra.py: every mechanism alone (the
kernels through their checked wrappers), then whole models built from folders that this file writes (its own small
configurations and weights), stepped through the engine in every way a request can arrive."""
import json
import math
import os

import pytest
import torch

import plain_sonodra as ps
from conftest import rel_err
from sonodra_cases import CONFIGS, _att, _dense, _lat, _moe, settled_tokens, write_folder

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
# Bounds on the distance from the plain implementation (float64 from the same stored weights).  float32: the largest
# difference of any element over the reference's root mean square: summation order and the float32 functions.
# bfloat16: activations are rounded to 8 bits at every part's boundary, which leaves a row's error near 1 % of its root
# mean square and single elements four to five times that; so a row's root-mean-square difference is bounded by 3 % and
# any element by 20 %.  A wrong key, a window one token off, a lost latent vector or another expert moves rows by their
# own size.
TOL = {torch.float32: 2e-4, torch.bfloat16: 3e-2}
BF16_ELEMENT = 0.2
DEV = "cuda:0"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """One folder a configuration, weights stored in bfloat16: engines of both types and the plain implementation read
    the same numbers."""
    made = {}

    def get(name):
        if name not in made:
            made[name] = write_folder(tmp_path_factory.mktemp(f"sonodra{name}"), CONFIGS[name], 11 + len(made))
        return made[name]
    return get


_plain_cache = {}


def plain(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        _plain_cache[key] = ps.forward(ps.read_config(folder), ps.read_weights(folder), tokens)
    return _plain_cache[key]


def engine(folder, dtype, max_tokens=1024, **kw):
    import bitnet_c_amd as bn
    return bn.Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, **kw)


def close(got, want, dtype, bf16_rows=None):
    e = rel_err(got, want)
    if dtype == torch.float32:
        assert e < TOL[dtype], f"relative error {e}"
        return
    g, w = got.detach().double().cpu().reshape(-1, got.shape[-1]), want.detach().double().cpu().reshape(-1, want.shape[-1])
    rms = float(w.pow(2).mean().sqrt())
    rows = float((g - w).pow(2).mean(dim=-1).sqrt().max()) / max(rms, 1e-30)
    assert rows < (bf16_rows or TOL[dtype]) and e < (10 * bf16_rows if bf16_rows else BF16_ELEMENT), \
        f"a row is {rows} rms off, an element {e}"


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [24, 256, 2500])
def test_an_output_with_its_own_norm_joins_the_stream(dtype, D):
    """x += w_b * d / rms(d), alone and together with the next norm, for an output in the activations' type and for one
    that arrives as float32 slabs still to be added."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(D)
    T, eps_b, eps = 7, 1e-5, 1e-6
    x0 = torch.randn(T, D, generator=g)
    d = (3.0 * torch.randn(T, D, generator=g)).to(dtype)
    slabs = torch.randn(3, T, D, generator=g)
    wb, w = 1 + 0.3 * torch.randn(D, generator=g), 1 + 0.3 * torch.randn(D, generator=g)
    for delta, dd in ((d.to(DEV), d.double()), (ops.PartialSums(slabs.to(DEV)), slabs.double().sum(0))):
        want_x = x0.double() + ps.unit_rms(dd, eps_b) * wb.double()
        x = x0.to(DEV).clone()
        assert ops.add_normed_rmsnorm(x, delta, wb.to(DEV), eps_b) is None
        assert rel_err(x, want_x) < 1e-5
        x = x0.to(DEV).clone()
        h = ops.add_normed_rmsnorm(x, delta, wb.to(DEV), eps_b, w.to(DEV), eps, dtype)
        assert h.dtype == dtype and rel_err(x, want_x) < 1e-5
        close(h, ps.unit_rms(want_x, eps) * w.double(), dtype)


def _split_half(x, positions, dims, base):
    """Pairs (i, i + dims / 2) turned by position * base^(-2i/dims): the other way of pairing, written out here (the angle
    rounded to float32, as the kernel forms it)."""
    out = x.clone()
    for t, p in enumerate(positions):
        for i in range(dims // 2):
            a = float(torch.tensor(float(p), dtype=torch.float32) * torch.tensor(float(base) ** (-2.0 * i / dims), dtype=torch.float32))
            u, v = x[t, :, i], x[t, :, i + dims // 2]
            out[t, :, i] = u * math.cos(a) - v * math.sin(a)
            out[t, :, i + dims // 2] = v * math.cos(a) + u * math.sin(a)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,hs,vd,rd", [(4, 2, 16, 24, 8), (6, 1, 8, 6, 2), (2, 2, 64, 64, 64), (3, 1, 130, 20, 128), (1, 1, 256, 256, 0)])
def test_projection_norms_rotation_and_the_cache_write(dtype, H, G, hs, vd, rd):
    """One norm over all query heads and one over all key heads, the rotation in neighbouring pairs (and in split-half
    pairs), the keys and values at their places in the pages; positions far apart, a padding row left alone."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    g = torch.Generator().manual_seed(H * 100 + hs)
    eps, base = 1e-5, 700.0
    pos = [0, 1, 63, 64, 300, -1, 2047]
    T = len(pos)
    qkv = torch.randn(T, H * hs + G * (hs + vd), generator=g).to(dtype)
    wq, wk = 1 + 0.2 * torch.randn(H * hs, generator=g), 1 + 0.2 * torch.randn(G * hs, generator=g)
    inv = torch.tensor([base ** (-2.0 * i / rd) for i in range(rd // 2)], dtype=torch.float32, device=DEV) if rd else None
    live = [t for t, p in enumerate(pos) if p >= 0]
    q = (ps.unit_rms(qkv[:, :H * hs].double(), eps) * wq.double()).view(T, H, hs)[live]
    k = (ps.unit_rms(qkv[:, H * hs:(H + G) * hs].double(), eps) * wk.double()).view(T, G, hs)[live]
    v = qkv[:, (H + G) * hs:].double().view(T, G, vd)[live]
    for interleaved in (True, False):
        if rd:
            rot = (lambda x, p, d, b: ps.rotate_pairs(x, p, d, b, angle_dtype=torch.float32)) if interleaved else _split_half
            qr, kr = rot(q, [pos[t] for t in live], rd, base), rot(k, [pos[t] for t in live], rd, base)
        else:
            qr, kr = q, k
        for transposed in (True, False):
            kp = torch.zeros(40, G, PAGE, hs, dtype=dtype, device=DEV)
            vp = torch.zeros((40, G, vd, PAGE) if transposed else (40, G, PAGE, vd), dtype=dtype, device=DEV)
            table = i32([[(7 * j + 3) % 40 for j in range(33)]])
            rows = qkv.to(DEV).clone()
            ops.qk_norm_store(rows, i32(pos), H, G, hs, v_dim=vd, q_weight=wq.to(DEV), k_weight=wk.to(DEV), eps=eps,
                              seq_index=i32([0] * T), block_table=table, k_pages=kp, v_pages=vp, v_transposed=transposed,
                              norm_projection=True, inv_freq=inv, rope_dims=rd, rope_interleaved=interleaved)
            tol = 3e-5 if dtype == torch.float32 else 2e-2          # the largest element's rounding over the root mean square
            assert rel_err(rows[live, :H * hs].view(-1, H, hs), qr) < tol
            assert torch.equal(rows[5], qkv[5].to(DEV))              # the padding row
            for n, t in enumerate(live):
                page, slot = int(table[0, pos[t] // PAGE]), pos[t] % PAGE
                assert rel_err(kp[page, :, slot], kr[n]) < tol
                got_v = vp[page, :, :, slot] if transposed else vp[page, :, slot]
                assert torch.equal(got_v.double().cpu(), v[n])
            assert int((kp != 0).any(dim=-1).sum()) == len(live) * G   # and nothing anywhere else


def _window_case(dtype, H, G, hs, vd, T, window, seed, spikes=(), scale=0.3):
    """Random queries, keys and values of one sequence, already normed and rotated; spikes: (query, key) pairs whose
    score is made to stand out (the key's value too).  Returns the pages' inputs and the plain result."""
    g = torch.Generator().manual_seed(seed)
    q, k, v = torch.randn(T, H, hs, generator=g), torch.randn(T, G, hs, generator=g), torch.randn(T, G, vd, generator=g)
    for i, j in spikes:
        if 0 <= j <= i:
            k[j] = 10.0 * q[i].view(G, H // G, hs)[:, 0] / scale / hs
            v[j] += 6.0
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).to(dtype)
    qd, kd = qkv[:, :H * hs].double().view(T, H, hs), qkv[:, H * hs:(H + G) * hs].double().view(T, G, hs)
    vd_ = qkv[:, (H + G) * hs:].double().view(T, G, vd)
    want = torch.zeros(T, H, vd, dtype=torch.float64)
    for t in range(T):
        first = max(0, t - window + 1) if window else 0
        for a in range(H):
            w = ps.softmax_over((kd[first:t + 1, a // (H // G)] @ qd[t, a]) * scale)
            want[t, a] = w @ vd_[first:t + 1, a // (H // G)]
    return qkv, want.reshape(T, H * vd)


def _run_window_case(dtype, H, G, hs, vd, T, window, qkv, scale, portions, matrix_cores):
    """The sequence through the kernels: `portions` as prompt steps (each reads the pages of those before it), the rest
    token by token."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    n_pages = -(-T // PAGE)
    g = torch.Generator().manual_seed(5)
    kp = torch.zeros(n_pages + 3, G, PAGE, hs, dtype=dtype, device=DEV)
    vp = torch.zeros(n_pages + 3, G, vd, PAGE, dtype=dtype, device=DEV)
    table = torch.randperm(n_pages + 3, generator=g)[:n_pages].to(torch.int32).view(1, -1).to(DEV).contiguous()
    outs, lo = [], 0
    for n in list(portions) + [1] * (T - sum(portions)):
        rows = qkv[lo:lo + n].to(DEV).contiguous()
        pos = torch.arange(lo, lo + n, dtype=torch.int32, device=DEV)
        ops.qk_norm_store(rows, pos, H, G, hs, v_dim=vd, seq_index=i32([0] * n), block_table=table, k_pages=kp, v_pages=vp,
                          v_transposed=True)
        out = torch.full((n, H * vd), 9.0, dtype=dtype, device=DEV)
        if n == 1 and lo > 0 and matrix_cores:
            n_splits, chunk, _ = ops.general_decode_plan(1, H, G, table.shape[1] * PAGE, window)      # for what the table can hold
            ops.attention_general_decode(rows, out, kp, vp, table, pos + 1, H, G, hs, vd, scale, window=window,
                                         n_splits=n_splits, chunk=chunk)
        elif n == 1 and lo > 0:
            n_splits, chunk = 1, 0
            if window >= 4 * PAGE and dtype == torch.bfloat16:      # a long window is cut from its own first page on
                n_splits, chunk = ops.decode_splits(1, H, G, window + PAGE, dtype, target_wgs=ops.VECTOR_DECODE_TARGET_WGS)
                assert n_splits > 1
            ops.attention(rows, out, kp, vp, table, H, G, hs, scale, window=window, seq_lens=pos + 1, n_splits=n_splits,
                          chunk=chunk, v_transposed=True, blocked=False, v_dim=vd)
        elif matrix_cores:
            qt = ops.GENERAL_PROMPT_TILE
            tiles = i32([[0, i, min(qt, n - i), lo + i] for i in range(0, n, qt)][::-1] + [[0, 0, 0, 0]])
            ops.attention_general_prompt(rows, out, kp, vp, table, H, G, hs, vd, scale, tiles, window=window)
        else:
            _, _, qt = ops.attention_row_shape(H, G, False)
            tiles = i32([[0, i, min(qt, n - i), lo + i] for i in range(0, n, qt)])
            ops.attention(rows, out, kp, vp, table, H, G, hs, scale, window=window, tiles=tiles, qt=qt, v_transposed=True,
                          blocked=False, v_dim=vd)
        outs.append(out)
        lo += n
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 2, 31, 64, 65, 100, 300])
def test_a_window_and_its_edges_on_the_vector_kernel(dtype, window):
    """Queries in prompt portions and decoded alone whose one outstanding key lies just inside the window (the oldest
    visible position) or just outside it (one older): the first must carry the result, the second must not be seen.  The
    long window's decode steps are cut into splits (bfloat16), which begin at the window's first page."""
    H, G, hs, vd, T, scale = 4, 2, 16, 24, 200 if window < 256 else 720, 0.3
    queries = [3, 64, 70, 127, 128, 129, 140, 160, 180, 199] + ([299, 300, 301, 383, 384, 450, 639, 640, 641, 719] if T > 200 else [])
    for inside in (True, False):
        spikes = [(i, i - window + (1 if inside else 0)) for i in queries]
        qkv, want = _window_case(dtype, H, G, hs, vd, T, window, 10 * window + inside, spikes, scale)
        got = _run_window_case(dtype, H, G, hs, vd, T, window, qkv, scale, (70, 80), False)
        close(got, want, dtype)


@pytest.mark.parametrize("H,G,hs,vd", [(4, 2, 64, 64), (3, 1, 32, 96), (2, 2, 128, 128)])
@pytest.mark.parametrize("window", [1, 17, 32, 33, 64, 100])
def test_a_window_and_its_edges_on_the_matrix_cores(H, G, hs, vd, window):
    T, scale, dtype = 200, 1.0 / math.sqrt(hs), torch.bfloat16
    queries = [3, 15, 16, 64, 70, 127, 128, 129, 140, 149, 150, 199]
    for inside in (True, False):
        spikes = [(i, i - window + (1 if inside else 0)) for i in queries]
        qkv, want = _window_case(dtype, H, G, hs, vd, T, window, 7 * window + inside + hs, spikes, scale)
        got = _run_window_case(dtype, H, G, hs, vd, T, window, qkv, scale, (70, 80), True)
        close(got, want, dtype)


@pytest.mark.parametrize("H,hs,T", [(16, 64, 330), (20, 256, 200), (5, 128, 700)])
def test_many_heads_over_one_kv_head_on_the_matrix_cores(H, hs, T):
    """No window, every head sharing the one kv head whose values are as wide as its keys (what a latent attention asks
    for): prompt portions, then tokens one by one through the decode form with its keys in splits; single far keys carry
    some of the queries."""
    dtype, scale = torch.bfloat16, 1.0 / math.sqrt(hs)
    spikes = [(i, j) for i, j in ((150, 0), (151, 63), (152, 64), (T - 1, 1), (T - 2, 65), (T - 3, 127), (T - 4, T - 5)) if j <= i]
    qkv, want = _window_case(dtype, H, 1, hs, hs, T, 0, H + hs, spikes, scale)
    got = _run_window_case(dtype, H, 1, hs, hs, T, 0, qkv, scale, (70, 80), True)
    close(got, want, dtype)


def test_decode_on_the_matrix_cores_a_batch_with_a_padding_row_and_the_length_on_the_device():
    """Three rows of a decode step: a short sequence, a long one, a padding row (no keys: zeros); the keys per split
    follow the longest sequence's length, which lies in device memory; a sink and a distance bias as well."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    dtype, H, G, hs, vd, scale = torch.bfloat16, 6, 2, 32, 64, 0.2
    lens = [5, 300]
    g = torch.Generator().manual_seed(3)
    kp = torch.zeros(12, G, PAGE, hs, dtype=dtype, device=DEV)
    vp = torch.zeros(12, G, vd, PAGE, dtype=dtype, device=DEV)
    table = i32([[3, 0, 0, 0, 0, 0, 0, 0], [7, 1, 9, 4, 11, 0, 0, 0], [0, 0, 0, 0, 0, 0, 0, 0]])
    da, db = 0.3 * torch.rand(H, generator=g), 0.1 + torch.rand(H, generator=g)
    rows, wants = [], []
    for b, n in enumerate(lens):
        q, k, v = torch.randn(n, H, hs, generator=g), torch.randn(n, G, hs, generator=g), torch.randn(n, G, vd, generator=g)
        qkv = torch.cat([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)], 1).to(dtype)
        ops.qk_norm_store(qkv.to(DEV), i32(list(range(n))), H, G, hs, v_dim=vd, seq_index=i32([b] * n), block_table=table,
                          k_pages=kp, v_pages=vp, v_transposed=True)
        qd = qkv[-1, :H * hs].double().view(H, hs)
        kd, vd_ = qkv[:, H * hs:(H + G) * hs].double().view(n, G, hs), qkv[:, (H + G) * hs:].double().view(n, G, vd)
        o = torch.zeros(H, vd, dtype=torch.float64)
        for a in range(H):
            sc = (kd[:, a // (H // G)] @ qd[a]) * scale - float(da[a]) * torch.log1p(float(db[a]) * torch.arange(n - 1, -1, -1, dtype=torch.float64))
            e = torch.exp(sc - sc.max())
            o[a] = (e @ vd_[:, a // (H // G)]) / (e.sum() + math.exp(-float(sc.max())))      # the sink: one more term of score 0
        rows.append(qkv[-1])
        wants.append(o.reshape(-1))
    rows.append(torch.randn(H * hs + G * (hs + vd), generator=g).to(dtype))
    q = torch.stack(rows).to(DEV)
    for n_splits in (1, 4):
        out = torch.full((3, H * vd), 5.0, dtype=dtype, device=DEV)
        ops.attention_general_decode(q, out, kp, vp, table, i32(lens + [0]), H, G, hs, vd, scale, n_splits=n_splits,
                                     chunk=2 * PAGE, max_len_dev=i32([300]) if n_splits > 1 else None,
                                     distance_bias=(da.to(DEV), db.to(DEV)), sink=True)
        close(out[:2], torch.stack(wants), dtype)
        assert float(out[2].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,I,O,T", [(3, 16, 32, 5), (5, 12, 24, 40), (4, 64, 128, 16), (2, 128, 32, 100), (1, 20, 30, 1)])
def test_a_product_per_head(dtype, H, I, O, T):
    """y[t, h] = x[t, h] . M_h, from a strided view of a wider matrix, with and without the sigmoid gate; few rows (the
    kernel) and many (bf16: the library's batched product)."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(H * I + O)
    wide = torch.randn(T, H * I + 8, generator=g).to(dtype)
    w = (torch.randn(H, I, O, generator=g) / math.sqrt(I)).to(dtype)
    gate = torch.randn(T, H * O + 8, generator=g).to(dtype)
    want = torch.einsum("thi,hio->tho", wide[:, :H * I].double().view(T, H, I), w.double()).reshape(T, H * O)
    xd, gd = wide.to(DEV), gate.to(DEV)
    close(ops.head_linear(xd[:, :H * I], w.to(DEV)), want, dtype)
    close(ops.head_linear(xd[:, :H * I], w.to(DEV), gd[:, 8:]), want * ps.sigmoid(gate[:, 8:].double()), dtype)
    close(ops.head_linear(xd[:, :H * I], w.to(DEV), gd[:, 8:], allow_library=False), want * ps.sigmoid(gate[:, 8:].double()), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank", [8, 24, 128, 200])
def test_the_latent_vector_is_normed_and_stored_twice(dtype, rank):
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    g = torch.Generator().manual_seed(rank)
    pos, col, eps = [0, 63, 64, -1, 200], 10, 1e-5
    x = torch.randn(len(pos), col + rank + 3, generator=g).to(dtype)
    w = 1 + 0.2 * torch.randn(rank, generator=g)
    kp = torch.zeros(9, 1, PAGE, rank, dtype=dtype, device=DEV)
    vp = torch.zeros(9, 1, rank, PAGE, dtype=dtype, device=DEV)
    table = i32([[5, 2, 8, 1], [4, 0, 3, 7]])
    seq = [0, 1, 1, 0, 0]
    ops.latent_store(x.to(DEV), col, rank, w.to(DEV), eps, i32(pos), i32(seq), table, kp, vp)
    c = ps.unit_rms(x[:, col:col + rank].double(), eps) * w.double()
    for t, p in enumerate(pos):
        if p < 0:
            continue
        page = int(table[seq[t], p // PAGE])
        close(kp[page, 0, p % PAGE][None], c[t][None], dtype, bf16_rows=1e-2)
        assert torch.equal(vp[page, 0, :, p % PAGE], kp[page, 0, p % PAGE])
    assert int((kp != 0).any(dim=-1).sum()) == 4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,K,D", [(6, 2, 64), (3, 3, 48), (1, 1, 32), (70, 5, 40), (16, 1, 256)])
def test_the_router_chooses_the_largest_scores(dtype, E, K, D):
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(E * 10 + K)
    T = 50
    h = torch.randn(T, D, generator=g).to(dtype)
    r = (3.0 * torch.randn(E, D, generator=g) / math.sqrt(D)).to(torch.bfloat16).float()
    r[min(2, E - 1)] = r[0]                                  # two experts with equal scores: the lower index goes first
    z = h.double() @ r.double().T
    ids, wts = ops.moe_route(h.to(DEV), r.to(DEV), K)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))
        gap = float(z[t, order[K - 1]] - z[t, order[K]]) if K < E else 1.0
        if gap > 1e-3 and all(abs(float(z[t, a] - z[t, b])) > 1e-3 or {a, b} == {0, min(2, E - 1)}
                              for a in order[:K] for b in order[:K] if a < b):
            assert ids[t].tolist() == order[:K], t
            assert rel_err(wts[t], ps.sigmoid(z[t, order[:K]])) < 1e-5
    ids2, wts2 = ops.moe_route(h.to(DEV), r.to(DEV), K, "softmax", True)
    assert torch.equal(ids2, ids) and rel_err(wts2.sum(-1), torch.ones(T)) < 1e-5
    sm = torch.softmax(z, -1)
    pick = torch.gather(sm, 1, ids.long().cpu())
    assert rel_err(wts2, pick / pick.sum(-1, keepdim=True)) < 1e-4
    nan = torch.full((3, D), float("nan"), dtype=dtype, device=DEV)     # a padding row's garbage still names experts that exist
    ids3, _ = ops.moe_route(nan, r.to(DEV), K)
    assert int(ids3.min()) >= 0 and int(ids3.max()) < E


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,K,D,F,T", [(6, 2, 64, 32, 40), (3, 3, 48, 16, 9), (1, 1, 32, 8, 20), (9, 4, 96, 64, 70), (16, 1, 128, 64, 300), (4, 2, 72, 40, 700), (5, 1, 36, 20, 30)])
def test_the_experts_compute_on_the_weighted_input(dtype, E, K, D, F, T):
    """Every (token, choice) pair against expert(w h), summed over a token's choices; a pair a workgroup, and (bf16, rows
    of whole 16-byte groups) the grouped products over pairs ordered by expert; the weight on the output as well."""
    from bitnet_c_amd import ops
    g = torch.Generator().manual_seed(E + D + T)
    h = torch.randn(T, D, generator=g).to(dtype)
    up = (torch.randn(E, F, D, generator=g) / math.sqrt(D)).to(dtype)
    down = (torch.randn(E, D, F, generator=g) / math.sqrt(F)).to(dtype)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    if E > 2:
        ids[: T // 2, 0] = 1                                 # an expert with many rows (several tiles), others with none
        ids[: T // 2, 1:] = torch.stack([torch.tensor([e for e in torch.randperm(E, generator=g).tolist() if e != 1][:K - 1])
                                         for _ in range(T // 2)]).to(torch.int32).reshape(T // 2, K - 1)
    wts = torch.rand(T, K, generator=g) * 0.9 + 0.05
    W = {f"e{e}.up": up[e].double() for e in range(E)}
    W.update({f"e{e}.down": down[e].double() for e in range(E)})
    for on_input in (True, False):
        want = torch.zeros(T, D, dtype=torch.float64)
        for t in range(T):
            for j in range(K):
                e, w = int(ids[t, j]), float(wts[t, j])
                want[t] += ps.expert(w * h[t].double(), W, f"e{e}.") if on_input else w * ps.expert(h[t].double(), W, f"e{e}.")
        args = (h.to(DEV), up.to(DEV), down.to(DEV), ids.to(DEV), wts.to(DEV), "relu2", on_input)
        y = ops.moe_experts(*args)
        assert tuple(y.slabs.shape) == (K, T, D)
        close(y.slabs.sum(0), want, dtype)
        if ops.moe_grouped_supported(T, D, F, dtype):
            y = ops.moe_experts_grouped(*args)
            close(y.slabs.sum(0), want, dtype)
    assert ops.moe_grouped_supported(T, D, F, dtype) == (dtype == torch.bfloat16 and T >= 17 and D % 8 == 0 and F % 8 == 0)


# ------------------------------------------------------------------------------------------------------------------
# whole models through the engine
# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts_and_the_stream_after_every_layer(folders, name, dtype):
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype)
    for n in (1, 2, 77, 150):
        toks = settled_tokens(folder, n, 1)
        streams, got = [], []
        want = ps.forward(ps.read_config(folder), ps.read_weights(folder), toks, streams)
        eng.tap = lambda point, entry, stream, ctx: got.append(stream.flush().clone()) if point == "layer_out" else None
        s = eng.new_sequence()
        logits = eng.step([bn.StepEntry(s, toks, list(range(n)))])
        eng.release(s)
        eng.tap = None
        assert len(got) == len(streams) == len(CONFIGS[name]["layers"])
        for a, b in zip(got, streams):
            close(a, b, dtype)
        close(logits, want, dtype)
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prefill_against_decoding_token_by_token(folders, name, dtype, graphs):
    """A prompt, then 100 tokens one by one (across page borders and past every window), against the plain implementation
    of the whole sequence; and the same sequence from its very first token one by one."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype, use_graphs=graphs)
    toks = settled_tokens(folder, 150, 1)
    want = plain(folder, toks)
    for first in (50, 1):
        s = eng.new_sequence()
        parts = [eng.step([bn.StepEntry(s, toks[:first], list(range(first)))])]
        for t in range(first, len(toks) if first == 50 else 40):
            parts.append(eng.step([bn.StepEntry(s, [toks[t]], [0])]))
        eng.release(s)
        got = torch.cat(parts)
        close(got, want[:got.shape[0]], dtype)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_of_several_sizes(folders, name, dtype):
    """A prompt cut into portions of 2, 3, 1, 64, 5, 2, ... tokens gives what the whole prompt gives."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype)
    toks = settled_tokens(folder, 150, 1)
    want = plain(folder, toks)
    for cuts in ([2, 3, 1, 64, 5, 2, 40, 2, 31], [2] * 75, [149, 1], [63, 1, 1, 85]):
        assert sum(cuts) == len(toks)
        s, at, parts = eng.new_sequence(), 0, []
        for n in cuts:
            parts.append(eng.step([bn.StepEntry(s, toks[at:at + n], list(range(n)))]))
            at += n
        eng.release(s)
        close(torch.cat(parts), want, dtype)
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_unequal_batches_and_slots_used_again(folders, name, dtype, graphs):
    """Requests of 1, 70, 9 and 130 tokens as one batch, decoded together while the shorter ones end; then other
    requests in the slots and pages that were given back (windowed layers give pages back while a request still runs);
    every request against itself alone (the plain implementation)."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype, max_tokens=1024, use_graphs=graphs)
    for round_, lens in enumerate(([1, 70, 9, 130], [64, 3, 128], [5])):
        reqs = [settled_tokens(folder, n + 6 + 3 * i, 2 + (round_ + i) % 4) for i, n in enumerate(lens)]
        slots = [eng.new_sequence() for _ in reqs]
        got = [[] for _ in reqs]
        out = eng.step([bn.StepEntry(s, r[:n], [n - 1]) for s, r, n in zip(slots, reqs, lens)])
        for i in range(len(reqs)):
            got[i].append(out[i:i + 1])
        at = list(lens)
        live = list(range(len(reqs)))
        while live:
            out = eng.step([bn.StepEntry(slots[i], [reqs[i][at[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                got[i].append(out[j:j + 1])
                at[i] += 1
            for i in [i for i in live if at[i] == len(reqs[i])]:
                eng.release(slots[i])
                live.remove(i)
        for i, r in enumerate(reqs):
            close(torch.cat(got[i]), plain(folder, r)[lens[i] - 1:], dtype)
        eng.cache.check()
    assert eng.cache.live_slots() == []


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_steps_replayed_from_graphs(folders, name, dtype):
    """Prompt steps of one size run eagerly the first time, are recorded the second time and replayed afterwards, with
    other sequences in other slots each time: every one of them against the plain implementation, and what a recorded step
    left in the cache is what the tokens decoded behind it go on from."""
    import bitnet_c_amd as bn
    folder = folders(name)
    eng = engine(folder, dtype)
    assert eng.prompt_graphs
    keep = eng.new_sequence()                      # a live neighbour, so that later sequences get other slots
    eng.step([bn.StepEntry(keep, settled_tokens(folder, 9, 1), [])])
    for i in range(5):
        reqs = [settled_tokens(folder, n, 2 + (i + k) % 4) for k, n in enumerate((70 + i, 20 - i))]
        slots = [eng.new_sequence() for _ in reqs]
        out = eng.step([bn.StepEntry(s, r[:-3], [0, len(r) - 4]) for s, r in zip(slots, reqs)])
        tail = [eng.step([bn.StepEntry(s, [r[t]], [0]) for s, r in zip(slots, reqs)]) for t in (-3, -2, -1)]
        for k, r in enumerate(reqs):
            want = plain(folder, r)
            close(out[2 * k:2 * k + 2], want[[0, len(r) - 4]], dtype)
            close(torch.cat([t[k:k + 1] for t in tail]), want[-3:], dtype)
        eng.release(slots[i % 2])
    assert eng.graphs_built >= 2                   # a prompt step and the decode steps were recorded
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_that_mixes_single_tokens_and_portions(folders, dtype):
    import bitnet_c_amd as bn
    folder = folders("A")
    eng = engine(folder, dtype)
    a, b, c = (settled_tokens(folder, n, 2 + i) for i, n in enumerate((30, 90, 12)))
    sa, sb, sc = (eng.new_sequence() for _ in range(3))
    eng.step([bn.StepEntry(sa, a[:29], []), bn.StepEntry(sb, b[:10], [])])
    out = eng.step([bn.StepEntry(sa, a[29:], [0]), bn.StepEntry(sb, b[10:], [0, 79]), bn.StepEntry(sc, c, [11])])
    want = torch.stack([plain(folder, a)[29], plain(folder, b)[10], plain(folder, b)[89], plain(folder, c)[11]])
    close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_with_peaked_attentions(tmp_path, dtype):
    """A long sequence (past a run of a float32 cache's keys, many pages, windows that have left dozens of pages behind)
    whose attentions are peaked (large scales, so that single far latent vectors and single keys at a window's far end
    carry the result), as a prompt in portions and then decoded for 80 tokens."""
    import bitnet_c_amd as bn
    cfg = dict(architecture="Sonodra", vocab=61, width=32, norm=dict(eps=1e-5), layers=[
        _lat(2, 8, 8, 16, 1.5, _dense(48)), _att(2, 1, 8, 8, 1.5, 300, (10000.0, 4), None),
        _lat(3, 4, 8, 16, 2.0, None, kv_from=0), _att(2, 2, 8, 4, 1.0, 64, None, _dense(40))])
    folder = write_folder(tmp_path / "peaked", cfg, 9)
    g = torch.Generator().manual_seed(2)
    toks = torch.randint(0, 61, (2200,), generator=g).tolist()
    # positions and angles are float32 in the engine; at 2,000 tokens and under a peaked softmax that alone is seen in
    # float32 logits, so the plain implementation rounds them alike here
    want = ps.forward(ps.read_config(folder), ps.read_weights(folder), toks, angle_dtype=torch.float32)
    eng = engine(folder, dtype, max_tokens=4608)
    s, at, parts = eng.new_sequence(), 0, []
    check = [0, 1, 63, 64, 65, 299, 300, 301, 2047, 2048, 2049, 2119]
    for n in (1000, 1047, 73):
        w = [p - at for p in check if at <= p < at + n]
        parts.append(eng.step([bn.StepEntry(s, toks[at:at + n], w)]))
        at += n
    # bfloat16: scores reach 12 here, so the rounding of queries and keys to 8 bits moves a score by up to 0.1 and a
    # weight of the softmax by a tenth; a wrong or a lost key moves a row by its own size
    close(torch.cat(parts), want[check], dtype, bf16_rows=0.1)
    dec = torch.cat([eng.step([bn.StepEntry(s, [toks[t]], [0])]) for t in range(at, 2200)])
    close(dec, want[at:], dtype, bf16_rows=0.1)
    s2 = eng.new_sequence()                              # and the same positions from one step over the whole sequence
    whole = eng.step([bn.StepEntry(s2, toks, list(range(at, 2200)))])
    assert rel_err(dec, whole) < (1e-4 if dtype == torch.float32 else 1.0)
    if dtype == torch.bfloat16:
        close(dec, whole.double(), dtype, bf16_rows=0.1)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_do_not_depend_on_the_cut_or_the_batch(folders, dtype):
    """Whole, in portions, one by one and beside other requests: float32 logits agree to the last bits, bfloat16 within
    its rounding (steps of few rows and of many take different kernels for the experts and the per-head products)."""
    import bitnet_c_amd as bn
    folder = folders("C")
    eng = engine(folder, dtype)
    toks, other = settled_tokens(folder, 100, 1), settled_tokens(folder, 37, 3)
    s = eng.new_sequence()
    whole = eng.step([bn.StepEntry(s, toks, list(range(100)))])
    eng.release(s)
    s, o = eng.new_sequence(), eng.new_sequence()
    a = eng.step([bn.StepEntry(o, other, []), bn.StepEntry(s, toks[:37], list(range(37)))])
    b = eng.step([bn.StepEntry(s, toks[37:99], list(range(62)))])
    c = eng.step([bn.StepEntry(s, toks[99:], [0]), bn.StepEntry(o, [5], [])])
    got = torch.cat([a, b, c])
    if dtype == torch.float32:
        assert rel_err(got, whole) < 2e-5
    else:
        close(got, whole.double(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    """Greedy generation through load() and generate(), the scheduler batching three prompts two at a time.  float32: the
    plain implementation's tokens, as far as no expert choice along the way is a close call; bfloat16: every token that was
    chosen holds, where it was chosen, the plain implementation's largest logit within rounding (up to the first close
    expert choice of the sequence that the engine itself wrote)."""
    import bitnet_c_amd as bn
    folder = folders(name)
    llm = bn.load(folder, dtype="float32" if dtype == torch.float32 else "bfloat16", max_tokens=1024)
    prompts = [settled_tokens(folder, n, 2 + i) for i, n in enumerate((5, 66, 1))]
    got = llm.generate(prompts, max_new_tokens=12, temperature=0.0, stop_ids=(), batch_size=2)
    cfg, W = ps.read_config(folder), ps.read_weights(folder)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        margins = []
        logits = ps.forward(cfg, W, p + g, margins=margins)[len(p) - 1:-1]
        settled = 0                                        # generated tokens before the first close call
        while settled < 12 and margins[len(p) + settled - 1] >= (1e-3 if dtype == torch.float32 else 0.05):
            settled += 1
        rms = float(logits.pow(2).mean().sqrt())
        for i, tok in enumerate(g[:settled]):
            gap = float(logits[i].max() - logits[i, tok])
            assert gap <= (1e-4 if dtype == torch.float32 else 4e-2) * rms, (i, gap / rms)
    llm.engine.cache.check()
    assert llm.engine.cache.live_slots() == []


def test_command_line_and_trace_replay(folders, tmp_path):
    """The command line generates from a Sonodra folder (also one that it writes itself from a configuration file, with
    random weights), and the trace replay program steps one through a batch of prompts and single tokens."""
    import subprocess
    import sys
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = folders("D")                                   # one expert, or two with wide margins: no close calls
    cfg, W = ps.read_config(folder), ps.read_weights(folder)
    prompt = settled_tokens(folder, 8, 1)
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "bitnet"), folder, "--prompt-token-ids", ",".join(map(str, prompt)),
                        "-n", "6", "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--quiet"], capture_output=True, text=True,
                       timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    ids = [int(x) for x in [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0].split(",")]
    logits = ps.forward(cfg, W, prompt + ids)[len(prompt) - 1:-1]
    for i, tok in enumerate(ids):
        assert float(logits[i].max() - logits[i, tok]) <= 1e-4 * float(logits.pow(2).mean().sqrt())
    conf = tmp_path / "conf.json"
    conf.write_text(json.dumps(CONFIGS["B"]))
    made = str(tmp_path / "made")
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "bitnet"), made, "--random", str(conf), "--seed", "4",
                        "--prompt-token-ids", "1,2,3", "-n", "4", "--fp32", "--token-ids", "--quiet", "--repeat-penalty", "1.0"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    assert len([l for l in p.stderr.splitlines() if l and l[0].isdigit()][0].split(",")) == 4
    assert ps.read_config(made)["layers"] == CONFIGS["B"]["layers"]
    # trace replay: two requests that start together, then go on token by token; the shorter one ends earlier
    folder = folders("A")
    a, b = settled_tokens(folder, 40, 2), settled_tokens(folder, 7, 3)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:37], "want": [0, 29, 36]}, {"id": "b", "tokens": b[:5], "want": [4]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[37:38], "want": [0]}, {"id": "b", "tokens": b[5:6], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[38:39], "want": []}, {"id": "b", "tokens": b[6:], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[39:], "want": [0]}], "end": ["a"]}]
    for dtype, name in ((torch.float32, "float32"), (torch.bfloat16, "bfloat16")):
        out = tmp_path / ("out_" + name)
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", name,
                            "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                           capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-1500:]
        assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
        assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "2.f32", "3.f32"]
        la, lb = plain(folder, a), plain(folder, b)
        want_rows = {0: torch.stack([la[0], la[29], la[36], lb[4]]), 1: la[37:38], 2: lb[6:7], 3: la[39:40]}
        for i, w in want_rows.items():
            got = torch.from_numpy(np.fromfile(str(out / f"{i}.f32"), dtype="<f4").reshape(-1, 101))
            close(got, w, dtype)
