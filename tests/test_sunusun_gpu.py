"""The Sunusun architecture against the plain implementation of tests/plain_sunusun.py: every mechanism alone
(the kernels through their checked wrappers), then whole models built from folders that this file writes (its own
small configurations and weights), stepped through the engine in every way a request can arrive."""
import json
import math
import os

import pytest
import torch

import plain_sunusun as ps
from conftest import rel_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
# Bounds on the distance from the plain implementation (which computes in float64 from the same stored weights).
# float32: the largest difference of any element, over the reference's root mean square: summation order and the
# float32 functions.  bfloat16: activations are rounded to 8 bits at every part's boundary, which at these weights
# (matrices N(0, 1/in), peaked softmaxes) leaves a row's error near 1 % of its root mean square and single elements
# four to five times that; so a row's root-mean-square difference is bounded by 3 % and any element by 20 %.  A lost
# state, a shifted token or a wrong key moves rows by their own size.
TOL = {torch.float32: 2e-4, torch.bfloat16: 3e-2}
BF16_ELEMENT = 0.2


from sunusun_cases import CONFIGS, _par, _wkv, write_folder  # noqa: E402


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, dtype):
        # bf16 engines read bf16 weights; the plain implementation reads the same file, so both see the same numbers
        key = (name, dtype)
        if key not in made:
            made[key] = write_folder(tmp_path_factory.mktemp(f"sunusun{name}"), CONFIGS[name], 3 + len(made), dtype,
                                     name_rank=name != "Q")
        return made[key]
    return get


def engine(folder, dtype, max_tokens=1024, **kw):
    import bitnet_c_amd as bn
    return bn.Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, **kw)


def plain(folder, tokens):
    return ps.forward(ps.read_config(folder), ps.read_weights(folder), tokens)


def tokens_of(vocab, seed, n):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


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


# ------------------------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------

def _seq_tensors(lengths, starts, dev):
    """positions, seq_index, tiles (one a sequence) of a flattened step."""
    pos, seq, tiles, row = [], [], [], 0
    for s, (n, p0) in enumerate(zip(lengths, starts)):
        pos += list(range(p0, p0 + n))
        seq += [s] * n
        tiles.append([s, row, n, p0])
        row += n
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    return i32(pos), i32(seq), i32(tiles).reshape(-1, 4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_with_position_vector_and_row_kernels(dtype):
    from bitnet_c_amd import ops
    dev = "cuda:0"
    g = torch.Generator().manual_seed(1)
    for D in (10, 33):                                   # an odd width ends on a sine
        table = torch.randn(7, D, generator=g).to(dtype)
        toks = torch.tensor([3, 0, 6, 6], dtype=torch.int32, device=dev)
        pos = torch.tensor([0, 1, 700, 4095], dtype=torch.int32, device=dev)
        x = ops.embed_gather_sinusoid(table.to(dev), toks, pos, ops.sinusoid_frequencies(D, 10000.0).to(dev))
        want = table.double()[toks.cpu().long()] + ps.sinusoid(4096, D)[pos.cpu().long()]
        assert rel_err(x, want) < 3e-4               # float32 angles of up to 4,095 radians
    z = (3.0 * torch.randn(5, 24, generator=g)).to(dtype)
    close(ops.unary_act(z.to(dev), "gelu_erf"), ps.gelu_exact(z.double()), dtype)
    close(ops.unary_act(z.to(dev), "tanh"), torch.tanh(z.double()), dtype)
    a, b = torch.randn(6, 40, generator=g).to(dtype), (5 * torch.randn(6, 40, generator=g)).to(dtype)
    wa, wb = torch.rand(40, generator=g), torch.rand(40, generator=g)
    want = 0.5 * (ps.unit_rms(a.double(), 1e-5) * wa.double() + ps.unit_rms(b.double(), 1e-5) * wb.double())
    close(ops.rmsnorm_mean(a.to(dev), wa.to(dev), b.to(dev), wb.to(dev), 1e-5), want, dtype)
    lg = torch.randn(3, 50, generator=g).to(dev)
    want = lg.cpu().double() * 0.37
    ops.scale_(lg, 0.37)
    assert rel_err(lg, want) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d", [(2, 24), (1, 64), (3, 20), (1, 130), (2, 7)])
def test_wkv_pieces_alone(dtype, H, d):
    """Token shift, the recurrence and the head norm with its gate, for two sequences of a step, the second of which
    comes in two portions through its state; a third slot stays untouched."""
    from bitnet_c_amd import ops
    dev, D, eps = "cuda:0", 36, 1e-5
    g = torch.Generator().manual_seed(H * 100 + d)
    A = H * d
    lens = [9, 21]
    hs = [torch.randn(n, D, generator=g).to(dtype) for n in lens]
    mu = torch.rand(5, D, generator=g)
    r, k, v = ([(torch.randn(n, A, generator=g) * s).to(dtype) for n in lens] for s in (1.0, 0.5, 1.0))
    dd = [(-1.0 + torch.randn(n, A, generator=g)).to(dtype) for n in lens]
    gate = [torch.randn(n, A, generator=g).to(dtype) for n in lens]
    w0, u, nw = 0.3 * torch.randn(A, generator=g), 0.5 * torch.randn(A, generator=g), 1 + 0.1 * torch.randn(A, generator=g)
    n_state = ops.wkv_state_floats(H, d, d)          # the heads' matrices, rows rounded up as the kernel holds them
    state = torch.zeros(4, n_state + D, dtype=torch.float32, device=dev)
    state[3] = 7.0
    slots = torch.tensor([2, 0], dtype=torch.int32, device=dev)

    def run(parts, starts):
        """One step: parts[s] = rows of sequence s (may be empty for none)."""
        lengths = [p.stop - p.start for p in parts]
        pos, seq, tiles = _seq_tensors(lengths, starts, dev)
        cat = lambda xs: torch.cat([x[p] for x, p in zip(xs, parts)]).to(dev).contiguous()
        h = cat(hs)
        mixes = ops.token_shift(h, mu.to(dev), state[:, n_state:], pos, seq, slots)
        o = ops.wkv_scan(cat(r), cat(k), cat(v), cat(dd), w0.to(dev), u.to(dev), h, state, slots, H, d, d, tiles=tiles)
        y = ops.head_norm_gate(o, cat(gate), nw.to(dev), H, d, eps)
        return mixes, o, y

    m1, o1, y1 = run([slice(0, 9), slice(0, 13)], [0, 0])
    m2, o2, y2 = run([slice(0, 0), slice(13, 21)], [9, 13])
    # decode form: one more token for sequence 1 alone would need more rows; the prompt form with one row does the same
    for s, n in enumerate(lens):
        hd = hs[s].double()
        want_mix = torch.stack([ps.token_shift(hd, mu[i].double()) for i in range(5)])
        w = torch.exp(-torch.exp(dd[s].double() + w0.double())).view(n, H, d)
        want_o = ps.wkv_recurrence(r[s].double().view(n, H, d), k[s].double().view(n, H, d), v[s].double().view(n, H, d), w,
                                   u.double().view(H, d))
        want_y = ps.unit_rms(want_o, eps).reshape(n, A) * nw.double() * ps.silu(gate[s].double())
        if s == 0:
            got_mix, got_o, got_y = m1[:, :9], o1[:9], y1[:9]
        else:
            got_mix, got_o, got_y = torch.cat([m1[:, 9:], m2], 1), torch.cat([o1[9:], o2]), torch.cat([y1[9:], y2])
        close(got_mix, want_mix, dtype)
        assert rel_err(got_o, want_o.reshape(n, A)) < 2e-5            # float32 whatever the activations' type
        close(got_y, want_y, dtype)
    assert bool((state[3] == 7.0).all()) and bool((state[1] == 0).all())
    assert torch.equal(state[0, n_state:].cpu(), hs[1][-1].float())      # the last input row, for the next step's shift


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [33, 320])
def test_mingru_alone(dtype, W):
    from bitnet_c_amd import ops
    dev = "cuda:0"
    g = torch.Generator().manual_seed(W)
    lens = [1, 30]
    zxg = [(2 * torch.randn(n, 3 * W, generator=g)).to(dtype) for n in lens]
    bz, bx = torch.randn(W, generator=g), torch.randn(W, generator=g)
    state = torch.zeros(3, W, dtype=torch.float32, device=dev)
    slots = torch.tensor([1, 2], dtype=torch.int32, device=dev)
    _, _, tiles = _seq_tensors([1, 17], [0, 0], dev)
    y1 = ops.mingru_scan(torch.cat([zxg[0], zxg[1][:17]]).to(dev), bz.to(dev), bx.to(dev), state, slots, W, tiles=tiles)
    # then sequence 1 goes on alone, token by token, in the decode form (sequence 0's row is a padding row: length 0)
    ys = []
    for t in range(17, 30):
        lens_dev = torch.tensor([0, t + 1], dtype=torch.int32, device=dev)
        rows = torch.cat([torch.zeros(1, 3 * W, dtype=dtype), zxg[1][t:t + 1]]).to(dev)
        ys.append(ops.mingru_scan(rows, bz.to(dev), bx.to(dev), state, slots, W, seq_lens=lens_dev)[1:])
    for s, n in enumerate(lens):
        z = torch.sigmoid(zxg[s][:, :W].double() + bz.double())
        c = zxg[s][:, W:2 * W].double() + bx.double()
        cand = torch.where(c >= 0, c + 0.5, torch.sigmoid(c))
        S, want = torch.zeros(W, dtype=torch.float64), []
        for t in range(n):
            S = (1 - z[t]) * S + z[t] * cand[t]
            want.append(S * ps.silu(zxg[s][t, 2 * W:].double()))
        got = y1[:1] if s == 0 else torch.cat([y1[1:]] + ys)
        close(got, torch.stack(want), dtype)
    assert bool((state[0] == 0).all())


def _attention_case(dtype, H, G, hs, vd, lens, seed, scale=0.4, spike=None, transposed=False):
    """Random q, k, v for one sequence; returns what the kernels give for the whole prompt and the plain result.
    spike = (query position, key position): that pair's score is made to stand out."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    dev, eps, coef, every = "cuda:0", 1e-5, 0.25, 5
    g = torch.Generator().manual_seed(seed)
    T = lens
    q, k, v = torch.randn(T, H, hs, generator=g), torch.randn(T, G, hs, generator=g), torch.randn(T, G, vd, generator=g)
    if spike is not None:
        i, j = spike
        k[j] = q[i].view(G, H // G, hs)[:, 0] * 1.0            # after the head norms the pair's score is the largest by far
        v[j] += 5.0
    wq, wk = 1 + 0.1 * torch.randn(hs, generator=g), 1 + 0.1 * torch.randn(hs, generator=g)
    da, db = 0.3 * torch.rand(H, generator=g), 0.1 + torch.rand(H, generator=g)
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).to(dtype)
    # plain
    qd, kd, vd_ = (qkv[:, :H * hs].double().view(T, H, hs), qkv[:, H * hs:(H + G) * hs].double().view(T, G, hs),
                   qkv[:, (H + G) * hs:].double().view(T, G, vd))
    qn = ps.unit_rms(qd, eps) * wq.double() * ps.query_temperature(T, coef, every)[:, None, None]
    kn = ps.unit_rms(kd, eps) * wk.double()
    if dtype == torch.bfloat16:                      # the cache holds the normed keys, and the kernel reads the queries, in bfloat16
        qn, kn = qn.to(dtype).double(), kn.to(dtype).double()
    pos = torch.arange(T)
    vis = pos[:, None] >= pos[None, :]
    want = torch.zeros(T, H, vd, dtype=torch.float64)
    for h in range(H):
        s = (qn[:, h] @ kn[:, h // (H // G)].T) * scale - ps.distance_bias(T, float(da[h]), float(db[h]))
        want[:, h] = ps.sink_softmax(s, vis) @ vd_[:, h // (H // G)]
    want = want.reshape(T, H * vd)
    n_pages = -(-T // PAGE)
    kp = torch.zeros(n_pages + 3, G, PAGE, hs, dtype=dtype, device=dev)
    vp = torch.zeros((n_pages + 3, G, vd, PAGE) if transposed else (n_pages + 3, G, PAGE, vd), dtype=dtype, device=dev)
    table = (torch.randperm(n_pages + 3, generator=g)[:n_pages]).to(torch.int32).view(1, -1).to(dev).contiguous()
    args = dict(q_weight=wq.to(dev), k_weight=wk.to(dev), eps=eps, temp_coef=coef, temp_every=every)
    return dict(qkv=qkv, want=want, kp=kp, vp=vp, table=table, args=args, bias=(da.to(dev), db.to(dev)), scale=scale)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,hs,vd", [(4, 2, 16, 24), (3, 3, 8, 6), (6, 2, 10, 16), (2, 1, 64, 64), (1, 1, 12, 100)])
def test_attention_pieces_alone(dtype, H, G, hs, vd):
    """Head norms, temperature and the cache write, then the vector kernel with distance bias, sink and its own value
    width: a prompt of 150 tokens in two steps (the second reads the first's pages), then tokens one by one."""
    from bitnet_c_amd import ops
    dev, T = "cuda:0", 181
    c = _attention_case(dtype, H, G, hs, vd, T, seed=H * 1000 + hs)
    _, _, qt = ops.attention_row_shape(H, G, False)
    outs = []
    for lo, hi in ((0, 70), (70, 150)):
        n = hi - lo
        rows = c["qkv"][lo:hi].to(dev).contiguous()
        pos = torch.arange(lo, hi, dtype=torch.int32, device=dev)
        seq = torch.zeros(n, dtype=torch.int32, device=dev)
        ops.qk_norm_store(rows, pos, H, G, hs, v_dim=vd, seq_index=seq, block_table=c["table"], k_pages=c["kp"],
                          v_pages=c["vp"], **c["args"])
        tiles = torch.tensor([[0, i, min(qt, n - i), lo + i] for i in range(0, n, qt)], dtype=torch.int32, device=dev)
        out = torch.empty(n, H * vd, dtype=dtype, device=dev)
        ops.attention(rows, out, c["kp"], c["vp"], c["table"], H, G, hs, c["scale"], tiles=tiles, qt=qt, v_transposed=False,
                      blocked=False, v_dim=vd, distance_bias=c["bias"], sink=True)
        outs.append(out)
    for t in range(150, T):
        rows = c["qkv"][t:t + 1].to(dev).contiguous()
        pos = torch.tensor([t], dtype=torch.int32, device=dev)
        ops.qk_norm_store(rows, pos, H, G, hs, v_dim=vd, seq_index=torch.zeros(1, dtype=torch.int32, device=dev),
                          block_table=c["table"], k_pages=c["kp"], v_pages=c["vp"], **c["args"])
        out = torch.empty(1, H * vd, dtype=dtype, device=dev)
        n_splits, chunk = (1, 0) if t % 2 else ops.decode_splits(1, H, G, t + 1, dtype)
        ops.attention(rows, out, c["kp"], c["vp"], c["table"], H, G, hs, c["scale"], seq_lens=pos + 1, n_splits=n_splits,
                      chunk=chunk, v_transposed=False, blocked=False, v_dim=vd, distance_bias=c["bias"], sink=True)
        outs.append(out)
    close(torch.cat(outs), c["want"], dtype)


@pytest.mark.parametrize("H,G,hs,vd", [(4, 2, 64, 64), (2, 1, 128, 32), (3, 3, 32, 96), (5, 1, 96, 128), (2, 2, 256, 256)])
def test_general_prompt_attention_on_the_matrix_cores(H, G, hs, vd):
    """The bf16 prompt kernel for the same mixer (keys a row per position, values transposed): a prompt in two portions
    whose tiles end in partial ones, the second portion reading the first's pages, and the tokens decoded behind it by the
    vector kernel over the same pages."""
    from bitnet_c_amd import ops
    dev, T, dtype = "cuda:0", 181, torch.bfloat16
    c = _attention_case(dtype, H, G, hs, vd, T, seed=H * 1000 + hs + vd, scale=1.0 / math.sqrt(hs), transposed=True)
    outs = []
    for lo, hi in ((0, 70), (70, 150)):
        n = hi - lo
        rows = c["qkv"][lo:hi].to(dev).contiguous()
        pos = torch.arange(lo, hi, dtype=torch.int32, device=dev)
        ops.qk_norm_store(rows, pos, H, G, hs, v_dim=vd, seq_index=torch.zeros(n, dtype=torch.int32, device=dev),
                          block_table=c["table"], k_pages=c["kp"], v_pages=c["vp"], v_transposed=True, **c["args"])
        qt = ops.GENERAL_PROMPT_TILE
        tiles = [[0, i, min(qt, n - i), lo + i] for i in range(0, n, qt)] + [[0, 0, 0, 0]]        # and a tile of no rows
        tiles = torch.tensor(tiles[::-1], dtype=torch.int32, device=dev)                          # in any order
        out = torch.full((n, H * vd), 7.0, dtype=dtype, device=dev)
        ops.attention_general_prompt(rows, out, c["kp"], c["vp"], c["table"], H, G, hs, vd, c["scale"], tiles,
                                     distance_bias=c["bias"], sink=True)
        outs.append(out)
    for t in range(150, T):
        rows = c["qkv"][t:t + 1].to(dev).contiguous()
        pos = torch.tensor([t], dtype=torch.int32, device=dev)
        ops.qk_norm_store(rows, pos, H, G, hs, v_dim=vd, seq_index=torch.zeros(1, dtype=torch.int32, device=dev),
                          block_table=c["table"], k_pages=c["kp"], v_pages=c["vp"], v_transposed=True, **c["args"])
        out = torch.empty(1, H * vd, dtype=dtype, device=dev)
        ops.attention(rows, out, c["kp"], c["vp"], c["table"], H, G, hs, c["scale"], seq_lens=pos + 1, v_transposed=True,
                      blocked=False, v_dim=vd, distance_bias=c["bias"], sink=True)
        outs.append(out)
    close(torch.cat(outs), c["want"], dtype)


@pytest.mark.parametrize("key", [0, 1, 31, 32, 63, 64, 65, 2047, 2048, 2100])
def test_a_far_key_on_the_matrix_cores(key):
    """One key whose score stands out, at the first positions and at the borders of the kernel's blocks of 32 keys and of
    the pages, seen from the last tokens of a prompt of 2,113 tokens, with and without the sink."""
    from bitnet_c_amd import ops
    dev, H, G, hs, vd, T, dtype = "cuda:0", 2, 1, 32, 32, 2113, torch.bfloat16
    c = _attention_case(dtype, H, G, hs, vd, T, seed=key, scale=1.5, spike=(T - 1, key), transposed=True)
    rows = c["qkv"].to(dev).contiguous()
    pos = torch.arange(T, dtype=torch.int32, device=dev)
    ops.qk_norm_store(rows, pos, H, G, hs, v_dim=vd, seq_index=torch.zeros(T, dtype=torch.int32, device=dev),
                      block_table=c["table"], k_pages=c["kp"], v_pages=c["vp"], v_transposed=True, **c["args"])
    qt = ops.GENERAL_PROMPT_TILE
    tiles = torch.tensor([[0, i, min(qt, T - i), i] for i in range(0, T, qt)], dtype=torch.int32, device=dev)
    out = torch.empty(T, H * vd, dtype=dtype, device=dev)
    ops.attention_general_prompt(rows, out, c["kp"], c["vp"], c["table"], H, G, hs, vd, c["scale"], tiles,
                                 distance_bias=c["bias"], sink=True)
    close(out[-40:], c["want"][-40:], dtype, bf16_rows=0.05)
    close(out[:70], c["want"][:70], dtype, bf16_rows=0.05)
    assert float(out[-1].float().abs().max()) > 2.0              # the key's value (shifted by 5) dominates


def test_the_sink_alone_takes_weight_when_every_score_is_low():
    """One key with a score far below zero: the softmax's weight goes to the sink, which has no value, and the
    result is near zero; without the sink the one key would get all of it."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.cache import PAGE
    dev, hs = "cuda:0", 8
    q = torch.ones(1, hs)
    k, v = -torch.ones(1, hs), 3 * torch.ones(1, hs)
    for sink, want in ((True, 3.0 * math.exp(-16.0) / (1 + math.exp(-16.0))), (False, 3.0)):
        kp, vp = torch.zeros(1, 1, PAGE, hs, device=dev), torch.zeros(1, 1, PAGE, hs, device=dev)
        rows = torch.cat([q, k, v], 1).to(dev)
        zero = torch.zeros(1, dtype=torch.int32, device=dev)
        table = torch.zeros(1, 1, dtype=torch.int32, device=dev)
        ops.qk_norm_store(rows, zero, 1, 1, hs, seq_index=zero, block_table=table, k_pages=kp, v_pages=vp)
        out = torch.empty(1, hs, device=dev)
        ops.attention(rows, out, kp, vp, table, 1, 1, hs, 2.0, seq_lens=zero + 1, v_transposed=False, blocked=False, sink=sink)
        assert abs(float(out[0, 0]) - want) < 1e-6 * max(1.0, want) + 1e-9


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("key", [0, 1, 62, 63, 64, 65, 127, 128, 2046, 2047, 2048, 2049, 2110])
def test_a_far_key_that_stands_out(dtype, key):
    """One key whose score stands out, at the first positions, at page borders and around the border of a run of a
    float32 cache's keys, seen from the prompt's last token and from a token decoded behind it, with the keys of a
    decode step split or not."""
    from bitnet_c_amd import ops
    dev, H, G, hs, vd, T = "cuda:0", 2, 1, 16, 16, 2113
    c = _attention_case(dtype, H, G, hs, vd, T, seed=key, scale=2.5, spike=(T - 1, key))
    c2 = _attention_case(dtype, H, G, hs, vd, T, seed=key, scale=2.5, spike=(T - 2, key))
    _, _, qt = ops.attention_row_shape(H, G, False)
    for case, upto in ((c2, T - 1), (c, T - 1)):
        rows = case["qkv"][:upto].to(dev).contiguous()
        pos = torch.arange(upto, dtype=torch.int32, device=dev)
        seq = torch.zeros(upto, dtype=torch.int32, device=dev)
        ops.qk_norm_store(rows, pos, H, G, hs, v_dim=vd, seq_index=seq, block_table=case["table"], k_pages=case["kp"],
                          v_pages=case["vp"], **case["args"])
        if case is c2:                                   # the prompt's last token asks for the key
            tiles = torch.tensor([[0, i, min(qt, upto - i), i] for i in range(0, upto, qt)], dtype=torch.int32, device=dev)
            out = torch.empty(upto, H * vd, dtype=dtype, device=dev)
            ops.attention(rows, out, case["kp"], case["vp"], case["table"], H, G, hs, case["scale"], tiles=tiles, qt=qt,
                          v_transposed=False, blocked=False, v_dim=vd, distance_bias=case["bias"], sink=True)
            close(out[-8:], case["want"][upto - 8:upto], dtype)
            assert float(out[-1].float().abs().max()) > 2.0          # the key's value (shifted by 5) dominates
        else:                                            # a decoded token asks for it
            row = case["qkv"][T - 1:T].to(dev).contiguous()
            p1 = torch.tensor([T - 1], dtype=torch.int32, device=dev)
            ops.qk_norm_store(row, p1, H, G, hs, v_dim=vd, seq_index=seq[:1], block_table=case["table"], k_pages=case["kp"],
                              v_pages=case["vp"], **case["args"])
            for splits in (ops.decode_splits(1, H, G, T, dtype), (1, 0) if dtype == torch.bfloat16 else None):
                if splits is None:
                    continue
                out = torch.empty(1, H * vd, dtype=dtype, device=dev)
                ops.attention(row, out, case["kp"], case["vp"], case["table"], H, G, hs, case["scale"], seq_lens=p1 + 1,
                              n_splits=splits[0], chunk=splits[1], v_transposed=False, blocked=False, v_dim=vd,
                              distance_bias=case["bias"], sink=True)
                close(out, case["want"][T - 1:], dtype)
                assert float(out.float().abs().max()) > 2.0


# ------------------------------------------------------------------------------------------------------------------
# whole models through the engine
# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts_and_the_stream_after_every_layer(folders, name, dtype):
    import bitnet_c_amd as bn
    folder = folders(name, dtype)
    eng = engine(folder, dtype)
    vocab = CONFIGS[name]["vocab"]
    for n in (1, 2, 77, 200):
        toks = tokens_of(vocab, n, n)
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
    """A prompt, then 70 tokens one by one (across a page border), against the plain implementation of the whole
    sequence; and the same sequence from its very first token one by one."""
    import bitnet_c_amd as bn
    folder = folders(name, dtype)
    eng = engine(folder, dtype, use_graphs=graphs)
    toks = tokens_of(CONFIGS[name]["vocab"], 11, 120)
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
    """A prompt cut into portions of 2, 3, 1, 64, 5, 2, ... tokens gives what the whole prompt gives; in float32
    within the float32 tolerance of the plain implementation, which a lost state or a shifted token would break."""
    import bitnet_c_amd as bn
    folder = folders(name, dtype)
    eng = engine(folder, dtype)
    toks = tokens_of(CONFIGS[name]["vocab"], 5, 150)
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
    requests in the slots and pages that were given back; every request against itself alone (the plain implementation)."""
    import bitnet_c_amd as bn
    folder = folders(name, dtype)
    eng = engine(folder, dtype, max_tokens=1024, use_graphs=graphs)
    vocab = CONFIGS[name]["vocab"]
    for round_, lens in enumerate(([1, 70, 9, 130], [64, 3, 128], [5])):
        reqs = [tokens_of(vocab, 100 * round_ + i, n + 6 + 3 * i) for i, n in enumerate(lens)]
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
    other sequences in other slots each time: every one of them against the plain implementation, and the state that a
    recorded step left is what the tokens decoded behind it go on from."""
    import bitnet_c_amd as bn
    folder = folders(name, dtype)
    eng = engine(folder, dtype)
    vocab = CONFIGS[name]["vocab"]
    keep = eng.new_sequence()                      # a live neighbour, so that later sequences get other slots
    eng.step([bn.StepEntry(keep, tokens_of(vocab, 1, 9), [])])
    for i in range(5):
        reqs = [tokens_of(vocab, 300 + 10 * i + k, n) for k, n in enumerate((70 + i, 20 - i))]
        slots = [eng.new_sequence() for _ in reqs]
        out = eng.step([bn.StepEntry(s, r[:-3], [0, len(r) - 4]) for s, r in zip(slots, reqs)])
        tail = [eng.step([bn.StepEntry(s, [r[t]], [0]) for s, r in zip(slots, reqs)]) for t in (-3, -2, -1)]
        for k, r in enumerate(reqs):
            want = plain(folder, r)
            close(out[2 * k:2 * k + 2], want[[0, len(r) - 4]], dtype)
            close(torch.cat([t[k:k + 1] for t in tail]), want[-3:], dtype)
        if i % 2:
            eng.release(slots[0])
        else:
            eng.release(slots[1])
    assert not eng.prompt_graphs or eng.graphs_built >= 2          # a prompt step and the decode steps were recorded
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_that_mixes_single_tokens_and_portions(folders, dtype):
    import bitnet_c_amd as bn
    folder = folders("P", dtype)
    eng = engine(folder, dtype)
    a, b, c = (tokens_of(97, 40 + i, n) for i, n in enumerate((30, 90, 12)))
    sa, sb, sc = (eng.new_sequence() for _ in range(3))
    eng.step([bn.StepEntry(sa, a[:29], []), bn.StepEntry(sb, b[:10], [])])
    out = eng.step([bn.StepEntry(sa, a[29:], [0]), bn.StepEntry(sb, b[10:], [0, 79]), bn.StepEntry(sc, c, [11])])
    want = torch.stack([plain(folder, a)[29], plain(folder, b)[10], plain(folder, b)[89], plain(folder, c)[11]])
    close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_with_a_peaked_attention(tmp_path, dtype):
    """A long sequence (past a run of a float32 cache's keys, many pages) whose attention is peaked (a large scale, so
    that single far keys carry the result), as a prompt in portions and then decoded for 80 tokens."""
    import bitnet_c_amd as bn
    cfg = dict(architecture="Sunusun", vocab=61, width=32, norm=dict(eps=1e-5), logit_scale=2.0, layers=[
        _par(2, 1, 8, 8, 3.0, 0.3, 64, 24, ff=48), _wkv(2, 8, 4), _par(2, 2, 8, 4, 2.0, 0.0, 7, 16)])
    folder = write_folder(tmp_path / "peaked", cfg, 9, dtype)
    toks = tokens_of(61, 2, 2200)
    # positions and angles are float32 in the engine; at 2,000 tokens and under a peaked softmax that alone is seen in
    # float32 logits, so the plain implementation rounds them alike here
    want = ps.forward(ps.read_config(folder), ps.read_weights(folder), toks, angle_dtype=torch.float32)
    eng = engine(folder, dtype, max_tokens=4608)
    s, at, parts = eng.new_sequence(), 0, []
    check = [0, 1, 63, 64, 65, 2047, 2048, 2049, 2119]
    for n in (1000, 1047, 73):
        w = [p - at for p in check if at <= p < at + n]
        parts.append(eng.step([bn.StepEntry(s, toks[at:at + n], w)]))
        at += n
    # bfloat16: scores reach 3 * 8 here, so the rounding of the normed queries and keys to 8 bits moves a score by up
    # to 0.1 and a weight of the softmax by a tenth; a wrong or a lost key moves a row by its own size
    close(torch.cat(parts), want[check], dtype, bf16_rows=0.1)
    dec = torch.cat([eng.step([bn.StepEntry(s, [toks[t]], [0])]) for t in range(at, 2200)])
    close(dec, want[at:], dtype, bf16_rows=0.1)
    s2 = eng.new_sequence()                              # and the same positions from one step over the whole sequence
    whole = eng.step([bn.StepEntry(s2, toks, list(range(at, 2200)))])
    assert rel_err(dec, whole) < (1e-5 if dtype == torch.float32 else 1.0)
    if dtype == torch.bfloat16:
        close(dec, whole.double(), dtype, bf16_rows=0.1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_float32_logits_do_not_depend_on_the_cut(folders, dtype):
    """Whole, in portions, one by one and in a batch: float32 logits are equal but for the rounding of the recurrences'
    last bits, bfloat16 within its rounding."""
    import bitnet_c_amd as bn
    folder = folders("Q", dtype)
    eng = engine(folder, dtype)
    toks = tokens_of(131, 8, 100)
    other = tokens_of(131, 9, 37)
    s = eng.new_sequence()
    whole = eng.step([bn.StepEntry(s, toks, list(range(100)))])
    eng.release(s)
    s, o = eng.new_sequence(), eng.new_sequence()
    a = eng.step([bn.StepEntry(o, other, []), bn.StepEntry(s, toks[:37], list(range(37)))])
    b = eng.step([bn.StepEntry(s, toks[37:99], list(range(62)))])
    c = eng.step([bn.StepEntry(s, toks[99:], [0]), bn.StepEntry(o, [5], [])])
    got = torch.cat([a, b, c])
    tol = 1e-5 if dtype == torch.float32 else TOL[dtype]
    assert rel_err(got, whole) < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    import bitnet_c_amd as bn
    folder = folders(name, dtype)
    llm = bn.load(folder, dtype="float32" if dtype == torch.float32 else "bfloat16", max_tokens=1024)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(vocab, 70 + i, n) for i, n in enumerate((5, 66, 1))]
    got = llm.generate(prompts, max_new_tokens=12, temperature=0.0, stop_ids=(), batch_size=2)
    cfg, W = ps.read_config(folder), ps.read_weights(folder)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        if dtype == torch.float32:
            assert g == ps.generate(cfg, W, p, 12)
            continue
        logits = ps.forward(cfg, W, p + g)[len(p) - 1:-1]         # every token that was chosen, where it was chosen
        rms = float(logits.pow(2).mean().sqrt())
        for i, tok in enumerate(g):
            assert float(logits[i].max() - logits[i, tok]) <= 4e-2 * rms
    llm.engine.cache.check()
    assert llm.engine.cache.live_slots() == []


def test_command_line_and_trace_replay(folders, tmp_path):
    """The command line generates from a Sunusun folder (also one that it writes itself from a configuration file, with
    random weights), and the trace replay program steps one through portions and single tokens."""
    import subprocess
    import sys
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = folders("P", torch.float32)
    cfg, W = ps.read_config(folder), ps.read_weights(folder)
    prompt = [3, 1, 4, 1, 5, 9, 2, 6]
    want = ps.generate(cfg, W, prompt, 6)
    base = [sys.executable, os.path.join(root, "bin", "bitnet"), folder, "--prompt-token-ids", ",".join(map(str, prompt)),
            "-n", "6", "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--quiet"]
    for extra in ([], ["--no-prefill"]):
        p = subprocess.run(base + extra, capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-1500:]
        ids = [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0]
        assert [int(x) for x in ids.split(",")] == want, extra
    conf = tmp_path / "conf.json"
    conf.write_text(json.dumps(CONFIGS["R"]))
    made = str(tmp_path / "made")
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "bitnet"), made, "--random", str(conf), "--seed", "4",
                        "--prompt-token-ids", "1,2,3", "-n", "4", "--fp32", "--token-ids", "--quiet", "--repeat-penalty", "1.0"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    ids = [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0]
    assert [int(x) for x in ids.split(",")] == ps.generate(ps.read_config(made), ps.read_weights(made), [1, 2, 3], 4)
    # trace replay: two requests, the first in two portions, then both token by token; logits at the wanted places
    a, b = tokens_of(97, 1, 40), tokens_of(97, 2, 7)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[30:38], "want": [7]}, {"id": "b", "tokens": b[:5], "want": [4]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[38:39], "want": [0]}, {"id": "b", "tokens": b[5:6], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[39:], "want": [0]}, {"id": "b", "tokens": b[6:], "want": [0]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    la, lb = ps.forward(cfg, W, a), ps.forward(cfg, W, b)
    want_rows = {0: la[[0, 29]], 1: torch.stack([la[37], lb[4]]), 2: la[38:39], 3: torch.stack([la[39], lb[6]])}
    for i, w in want_rows.items():
        got = torch.from_numpy(np.fromfile(str(out / f"{i}.f32"), dtype="<f4").reshape(-1, 97))
        close(got, w, torch.float32)
