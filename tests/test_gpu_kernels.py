"""Each kernel alone against a plain float64 computation, at other sizes than the engine's."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def t(x, dtype=torch.float32):
    return torch.as_tensor(np.asarray(x)).to(DEV).to(dtype).contiguous()


def bf16(x):
    return torch.as_tensor(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).float().numpy()


@pytest.mark.parametrize("T,N,K", [(1, 1, 1), (1, 37, 33), (3, 130, 31), (5, 64, 1025), (17, 151, 96), (64, 100, 70),
                                   (77, 300, 129), (200, 96, 224), (130, 257, 511), (129, 257, 200), (300, 331, 240),
                                   (513, 1152, 896), (2, 896, 4864), (40, 640, 1000), (64, 151, 72), (1000, 130, 136),
                                   (130, 257, 64), (200, 96, 192), (129, 300, 1024), (1000, 130, 128), (300, 331, 320),
                                   (700, 896, 4864), (65, 2100, 448),
                                   (300, 4608, 3584), (40, 3584, 18944), (24, 3584, 3584), (520, 9728, 896),
                                   (1100, 13400, 192),    # blocks of 384 tokens save a round of blocks
                                   # blocks of 256 x 160 fill the chip where 256 x 256 do not; the second with K in two
                                   (2000, 5000, 1088), (777, 5000, 3584),
                                   # many tokens by few rows; the second with K in four
                                   (1100, 900, 1088), (2000, 130, 2432),
                                   # few tiles and a long K
                                   (256, 896, 896), (130, 100, 1088), (200, 1152, 576), (300, 896, 2432),
                                   # one and two steps of the float32 tiles (K of 32 and 64), and every float32 block shape
                                   (40, 70, 32), (300, 100, 64), (2048, 9728, 96), (2048, 896, 160), (700, 300, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_all_modes_odd_sizes(T, N, K, dtype):
    from sprout_lm_amd import ops
    rng = np.random.default_rng(T * 1000 + N + K)
    a, w, b = rng.standard_normal((T, K)), rng.standard_normal((N, K)) / math.sqrt(K), rng.standard_normal(N)
    if dtype == torch.bfloat16:
        a, w, b = bf16(a), bf16(w), bf16(b)
    want = a.astype(np.float64) @ w.astype(np.float64).T
    tol = 1e-5 * max(1, math.sqrt(K) / 8) if dtype == torch.float32 else 2e-2
    A, W, B = t(a, dtype), t(w, dtype), t(b, dtype)
    out = torch.empty(T, N, dtype=dtype, device=DEV)
    ops.gemm(A, W, out, bias=B)
    assert np.abs(out.float().cpu().numpy() - (want + b)).max() <= tol * (1 + np.abs(want).max())
    out32 = torch.empty(T, N, dtype=torch.float32, device=DEV)
    ops.gemm(A, W, out32)                                   # float32 result of bfloat16 operands is not rounded
    assert np.abs(out32.cpu().numpy() - want).max() <= 1e-5 * max(1, math.sqrt(K) / 8) * (1 + np.abs(want).max())
    base = rng.standard_normal((T, N)).astype(np.float32)
    acc = t(base)
    ops.gemm(A, W, acc, accumulate=True)                    # the residual sum is float32
    assert np.abs(acc.cpu().numpy() - (base + want)).max() <= 1e-5 * max(1, math.sqrt(K) / 8) * (1 + np.abs(want).max())


# One product for every block shape of the tiled kernel, whole and with K split: (accumulate, T, N, K) -> (block rows,
# block columns, waves, K split?).  The plan is asserted, so that a change of the cost model that moves a size to
# another shape says so here instead of leaving a shape without a test.
BLOCK_SHAPE_SIZES = {
    (0, 65, 130, 64): (64, 64, 4, False), (1, 260, 130, 3584): (64, 64, 4, True),
    (0, 130, 13400, 64): (64, 128, 4, False), (1, 260, 2000, 18944): (64, 128, 4, True),
    (0, 264, 7000, 64): (128, 128, 8, False), (1, 65, 4608, 3584): (128, 128, 8, True),
    (0, 1024, 4608, 448): (256, 128, 8, False), (1, 200, 2570, 18944): (256, 128, 8, True),
    (0, 2056, 3590, 1088): (256, 160, 4, False), (1, 4104, 900, 9728): (256, 160, 4, True),
    (0, 513, 13400, 64): (256, 256, 8, False), (1, 1034, 4030, 9728): (256, 256, 8, True),
    (0, 1100, 13400, 64): (384, 256, 8, False), (1, 260, 13400, 9728): (384, 256, 8, True),
}


@pytest.mark.parametrize("case", sorted(BLOCK_SHAPE_SIZES))
def test_tiled_product_on_every_block_shape(case):
    from sprout_lm_amd import ops
    accumulate, T, N, K = case
    rows, cols, splits, waves = ops.pipe_plan(ops.PLAN_ACCUMULATE if accumulate else ops.PLAN_STORE, T, N, K)
    assert (rows, cols, waves, splits > 1) == BLOCK_SHAPE_SIZES[case], "this size has moved to another block shape"
    gen = torch.Generator(device=DEV).manual_seed(T + N)
    x = torch.randn(T, K, device=DEV, generator=gen).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV, generator=gen) * K ** -0.5).to(torch.bfloat16)
    want = x.float() @ w.float().T          # float32 product of the same bfloat16 operands
    if accumulate:
        before = torch.randn(T, N, device=DEV, generator=gen)
        out = before.clone()
        ops.gemm(x, w, out, accumulate=True)
        err = (out - (before + want)).abs().max().item()
        assert err <= 2e-5 * max(1.0, math.sqrt(K) / 8) * (1 + want.abs().max().item()), err
    else:
        bias = torch.randn(N, device=DEV, generator=gen).to(torch.bfloat16)
        out = torch.empty(T, N, dtype=torch.bfloat16, device=DEV)
        ops.gemm(x, w, out, bias=bias)
        want = want + bias.float()
        err = (out.float() - want).abs().max().item()
        assert err <= 2 ** -7 * (1 + want.abs().max().item()), err


@pytest.mark.parametrize("T,N,K", [(8, 151, 96), (16, 64, 1024), (7, 2050, 132), (13, 33, 4), (1, 896, 4864), (16, 1, 260)])
@pytest.mark.parametrize("a_dtype,w_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                             (torch.bfloat16, torch.float32)])
def test_gemm_float32_sums_for_few_tokens(T, N, K, a_dtype, w_dtype):
    """Up to 16 tokens with K in fours: the kernel whose waves own rows of the weights (odd N, one row, all modes)."""
    from sprout_lm_amd import ops
    rng = np.random.default_rng(T + N + K)
    a, w, b = rng.standard_normal((T, K)), rng.standard_normal((N, K)) / math.sqrt(K), rng.standard_normal(N)
    a = bf16(a) if a_dtype == torch.bfloat16 else a.astype(np.float32)
    w = bf16(w) if w_dtype == torch.bfloat16 else w.astype(np.float32)
    want = a.astype(np.float64) @ w.astype(np.float64).T
    tol = 1e-5 * max(1, math.sqrt(K) / 8) * (1 + np.abs(want).max())
    out = torch.full((T, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.gemm(t(a, a_dtype), t(w, w_dtype), out, bias=t(b.astype(np.float32)))
    assert np.abs(out.cpu().numpy() - (want + b)).max() <= tol
    base = rng.standard_normal((T, N)).astype(np.float32)
    acc = t(base)
    ops.gemm(t(a, a_dtype), t(w, w_dtype), acc, accumulate=True)
    assert np.abs(acc.cpu().numpy() - (base + want)).max() <= tol


@pytest.mark.parametrize("T,I,K", [(1, 16, 64), (8, 4864, 896), (16, 37, 132), (5, 40000, 64), (3, 100, 4864)])
def test_gated_product_of_few_tokens_in_float32(T, I, K):
    from sprout_lm_amd import ops
    rng = np.random.default_rng(T + I + K)
    x = rng.standard_normal((T, K)).astype(np.float32)
    w = (rng.standard_normal((2 * I, K)) * 2 / math.sqrt(K)).astype(np.float32)
    gate, up = x.astype(np.float64) @ w[:I].astype(np.float64).T, x.astype(np.float64) @ w[I:].astype(np.float64).T
    want = gate / (1 + np.exp(-gate)) * up
    out = torch.full((T, I), float("nan"), dtype=torch.float32, device=DEV)
    assert ops.gate_up_silu_f32(t(w), t(x), out)
    assert np.abs(out.cpu().numpy() - want).max() <= 1e-5 * max(1, math.sqrt(K) / 8) * (1 + np.abs(want).max())
    assert not ops.gate_up_silu_f32(t(w), t(np.zeros((17, K), np.float32)), torch.empty(17, I, device=DEV))    # more tokens: not taken


def test_gemm_mixed_operand_dtypes_and_refusals():
    from sprout_lm_amd import ops
    rng = np.random.default_rng(0)
    a, w = bf16(rng.standard_normal((9, 40))), rng.standard_normal((21, 40)).astype(np.float32)
    out = torch.empty(9, 21, dtype=torch.float32, device=DEV)
    ops.gemm(t(a, torch.bfloat16), t(w), out)               # a weight stored in 32-bit stays so
    assert np.abs(out.cpu().numpy() - a.astype(np.float64) @ w.astype(np.float64).T).max() < 1e-4
    with pytest.raises(ops.KernelError):
        ops.gemm(t(a, torch.bfloat16), t(w[:, :39]), out)
    with pytest.raises(ops.KernelError):
        ops.gemm(t(a, torch.bfloat16).cpu(), t(w), out)     # no CPU path
    with pytest.raises(ops.KernelError):
        ops.gemm(t(a, torch.bfloat16), t(w), torch.empty(9, 21, dtype=torch.bfloat16, device=DEV), accumulate=True)


@pytest.mark.parametrize("H", [1, 24, 96, 896, 1000, 5120])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(H, out_dtype):
    from sprout_lm_amd import ops
    rng = np.random.default_rng(H)
    x = (rng.standard_normal((7, H)) * 3).astype(np.float32)
    w = rng.uniform(0.5, 1.5, H).astype(np.float32)
    for eps in (1e-6, 1e-2):
        want = x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + eps) * w
        out = torch.empty(7, H, dtype=out_dtype, device=DEV)
        ops.rmsnorm(t(x), t(w), eps, out)
        tol = 2e-6 if out_dtype == torch.float32 else 2 ** -8
        assert np.abs(out.float().cpu().numpy() - want).max() <= tol * (1 + np.abs(want).max())
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    out = torch.empty(3, H, dtype=torch.float32, device=DEV)
    ops.rmsnorm(t(x), t(w), 1e-6, out, rows=rows)
    full = torch.empty(7, H, dtype=torch.float32, device=DEV)
    ops.rmsnorm(t(x), t(w), 1e-6, full)
    assert torch.equal(out, full[[5, 0, 5]])
    zero = torch.empty(2, H, dtype=torch.float32, device=DEV)
    ops.rmsnorm(torch.zeros(2, H, device=DEV), t(w), 1e-6, zero)
    assert torch.all(zero == 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_and_silu_mul(dtype):
    from sprout_lm_amd import ops
    rng = np.random.default_rng(1)
    table = rng.standard_normal((331, 70)).astype(np.float32)
    tokens = torch.tensor([330, 0, 7, 7, 128], dtype=torch.int32, device=DEV)
    res = torch.empty(5, 70, dtype=torch.float32, device=DEV)
    ops.embed(t(table, dtype), tokens, res)
    assert torch.equal(res, t(table, dtype).float()[tokens.long()])
    gu = rng.standard_normal((6, 2 * 333)).astype(np.float32) * 4
    if dtype == torch.bfloat16:
        gu = bf16(gu)
    g, u = gu[:, :333].astype(np.float64), gu[:, 333:].astype(np.float64)
    out = torch.empty(6, 333, dtype=dtype, device=DEV)
    ops.silu_mul(t(gu, dtype), out)
    want = g / (1 + np.exp(-g)) * u
    tol = 1e-6 if dtype == torch.float32 else 2 ** -8
    assert np.abs(out.float().cpu().numpy() - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_random_fill_equals_its_host_twin_bit_by_bit(dtype):
    """Random weights drawn on the device are the numbers that the host draws for the same (seed, name, index):
    a model folder written on the host and an engine that draws its weights on the GPU hold the same model."""
    from sprout_lm_amd import ops
    from sprout_lm_amd.weights.random_init import fill_numpy, key_for, random_tensors
    from sprout_lm_amd.weights import TensorSpec
    for name, n, first, offset in (("a", 1, 0, None), ("model.embed_tokens.weight", 100_003, 0, None),
                                   ("b.norm", 4099, 0, 1.0), ("c", 70_001, 5_000_000_123, None)):
        key = key_for(17, name)
        got = torch.empty(n, dtype=dtype, device=DEV)
        ops.random_fill(got, key, 0.02 / 65536, offset, first)
        want = torch.from_numpy(fill_numpy(key, n, 0.02 / 65536, offset, first)).to(dtype)
        assert torch.equal(got.cpu(), want), name
    expected = {"w": TensorSpec((37, 129)), "n": TensorSpec((129,), "vector", "one_plus_normal")}
    host, device = random_tensors(expected, 3, dtype, "cpu", 0.05), random_tensors(expected, 3, dtype, DEV, 0.05)
    assert all(torch.equal(host[k], device[k].cpu()) for k in expected)


def plain_rope(x, pos, hd, rotary, theta):
    x = x.astype(np.float64).copy()
    half = rotary // 2
    heads = x.shape[1] // hd
    d = np.arange(half)
    ang = pos[:, None] * theta ** (-2.0 * d / rotary)
    for h in range(heads):
        a, b = x[:, h * hd:h * hd + half].copy(), x[:, h * hd + half:h * hd + rotary].copy()
        x[:, h * hd:h * hd + half] = a * np.cos(ang) - b * np.sin(ang)
        x[:, h * hd + half:h * hd + rotary] = b * np.cos(ang) + a * np.sin(ang)
    return x


@pytest.mark.parametrize("nq,nkv,hd,rotary,page", [(4, 2, 16, 16, 16), (3, 1, 32, 32, 8), (5, 5, 48, 48, 4), (7, 1, 64, 32, 32),
                                                   (2, 2, 128, 128, 16), (1, 1, 6, 6, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_and_cache_write(nq, nkv, hd, rotary, page, dtype):
    from sprout_lm_amd import ops
    rng = np.random.default_rng(nq * 100 + hd)
    T, pages, theta = 11, 9, 10000.0
    qkv = rng.standard_normal((T, (nq + 2 * nkv) * hd)).astype(np.float32)
    if dtype == torch.bfloat16:
        qkv = bf16(qkv)
    pos = rng.integers(0, 500, T)
    slots = rng.permutation(pages * page)[:T].astype(np.int32)
    slots[3] = -1                                           # a token whose keys are not written
    inv = torch.tensor(theta ** (-2.0 * np.arange(rotary // 2) / rotary), dtype=torch.float32, device=DEV)
    Q = t(qkv, dtype)
    kp = torch.zeros(pages, nkv, page, hd, dtype=dtype, device=DEV)
    vp = torch.zeros(pages, nkv, hd, page, dtype=dtype, device=DEV)
    ops.rope_cache(Q, torch.tensor(pos, dtype=torch.int32, device=DEV), inv, rotary, nq, nkv, hd,
                   torch.tensor(slots, device=DEV), kp, vp)
    want_qk = plain_rope(qkv[:, :(nq + nkv) * hd], pos, hd, rotary, theta)
    tol = 2e-4 if dtype == torch.float32 else 2 ** -7       # float32 angles of positions up to 500
    got = Q.float().cpu().numpy()
    assert np.abs(got[:, :(nq + nkv) * hd] - want_qk).max() <= tol * 4
    assert np.array_equal(got[:, (nq + nkv) * hd:], qkv[:, (nq + nkv) * hd:])
    kp, vp = kp.float().cpu().numpy(), vp.float().cpu().numpy().transpose(0, 1, 3, 2)   # values lie [.., dim, slot]
    written = np.zeros((pages, page), bool)
    for i in range(T):
        if slots[i] < 0:
            continue
        pg, off = divmod(int(slots[i]), page)
        written[pg, off] = True
        for g in range(nkv):
            assert np.array_equal(kp[pg, g, off], got[i, (nq + g) * hd:(nq + g + 1) * hd])
            assert np.array_equal(vp[pg, g, off], qkv[i, (nq + nkv + g) * hd:(nq + nkv + g + 1) * hd])
    unwritten = ~written[:, None, :, None]                   # pools are [pages, groups, page, head size]
    assert np.all((kp == 0) | ~unwritten) and np.all((vp == 0) | ~unwritten)


def plain_attention(q, keys, values, nq, nkv, hd, first_pos, window, scale):
    """q [n, nq*hd] at positions first_pos..; keys/values [ctx, nkv*hd]."""
    out = np.zeros_like(q, dtype=np.float64)
    for i in range(q.shape[0]):
        p = first_pos + i
        lo = 0 if not window else max(0, p - window + 1)
        for h in range(nq):
            g = h // (nq // nkv)
            s = keys[lo:p + 1, g * hd:(g + 1) * hd] @ q[i, h * hd:(h + 1) * hd] * scale
            e = np.exp(s - s.max())
            out[i, h * hd:(h + 1) * hd] = (e / e.sum()) @ values[lo:p + 1, g * hd:(g + 1) * hd]
    return out


def run_attention(dtype, nq, nkv, hd, page, seqs, window=None, kind=0, spike=None, seed=0, hidden=None, exact_table=False,
                  poison=None):
    """seqs: list of (ctx_len, q_len).  Pages are scattered over the pool in random order.

    exact_table: a table row holds the longest sequence's pages and no entry more.  poison: a sequence whose pages
    are filled with NaN after the expected values have been taken (its own rows of the result mean nothing).

    hidden: an output projection [hidden, nq * hd] is given along, which the kernels must fold in; what is
    compared is then what was added to a float32 residual."""
    from sprout_lm_amd import ops
    rng = np.random.default_rng(seed)
    n_pages = sum(-(-c // page) for c, _ in seqs) + 3
    order = list(rng.permutation(n_pages))
    kp = rng.standard_normal((n_pages, nkv, page, hd)).astype(np.float32)     # unused slots hold noise, not zeros
    vp = rng.standard_normal((n_pages, nkv, page, hd)).astype(np.float32)
    if dtype == torch.bfloat16:
        kp, vp = bf16(kp), bf16(vp)
    T = sum(q for _, q in seqs)
    q = rng.standard_normal((T, nq * hd)).astype(np.float32)
    max_blocks = max(-(-c // page) for c, _ in seqs) + (0 if exact_table else 1)
    tables = np.full((len(seqs), max_blocks), -1, np.int32)
    keys, values, starts = [], [], []
    t0 = 0
    for s, (ctx, qlen) in enumerate(seqs):
        blocks = [order.pop() for _ in range(-(-ctx // page))]
        tables[s, :len(blocks)] = blocks
        k = np.concatenate([kp[b].transpose(1, 0, 2).reshape(page, nkv * hd) for b in blocks])[:ctx]
        v = np.concatenate([vp[b].transpose(1, 0, 2).reshape(page, nkv * hd) for b in blocks])[:ctx]
        if spike is not None and s == spike[0]:
            # one far key stands out for the last query: its score dominates, so missing it shows
            _, far = spike
            k[far] *= 0.0
            k[far, :hd] = 6.0
            q[t0 + qlen - 1, :] = 0.0
            for h in range(nq):
                q[t0 + qlen - 1, h * hd:h * hd + hd] = 3.0 if h // (nq // nkv) == 0 else 0.1
            pg, off = divmod(far, page)
            kp[blocks[pg], :, off, :] = k[far].reshape(nkv, hd)
        if dtype == torch.bfloat16:
            k, v = bf16(k), bf16(v)
        keys.append(k); values.append(v); starts.append(t0)
        t0 += qlen
        if poison == s:
            kp[blocks], vp[blocks] = np.nan, np.nan
    if dtype == torch.bfloat16:
        q, kp = bf16(q), bf16(kp)
    out = torch.full((T, nq * hd), float("nan"), dtype=dtype, device=DEV)
    scale = 1 / math.sqrt(hd)
    batch = ops.AttentionBatch.build([ql for _, ql in seqs], [c for c, _ in seqs], DEV)
    project = None
    if hidden:
        w_o = bf16(rng.standard_normal((hidden, nq * hd)).astype(np.float32) / math.sqrt(nq * hd))
        before = rng.standard_normal((T, hidden)).astype(np.float32)
        project = (t(w_o, dtype), t(before, torch.float32))
    folded = ops.attention(t(q, dtype), nq * hd, t(kp, dtype), t(vp.transpose(0, 1, 3, 2), dtype), t(tables, torch.int32),
                           batch, out, nq, nkv, hd, window, scale, kind=kind, project=project)
    want = np.concatenate([plain_attention(q[starts[s]:starts[s] + ql].astype(np.float64), keys[s].astype(np.float64),
                                           values[s].astype(np.float64), nq, nkv, hd, c - ql, window, scale)
                           for s, (c, ql) in enumerate(seqs)])
    if hidden and len(seqs) <= 32:
        assert folded, "the projection was not folded in"
        got = project[1].cpu().numpy().astype(np.float64) - before
        return got, bf16(want.astype(np.float32)).astype(np.float64) @ w_o.astype(np.float64).T
    # more sequences than the folding kernel takes: it declines, the residual is untouched and the attention's own
    # output is what is compared
    assert not folded
    if hidden:
        assert np.array_equal(project[1].cpu().numpy(), before)
    got = out.float().cpu().numpy()
    return got, want


# (4, 2, 64, 12) and (5, 1, 48, 6): pages whose size is no power of two (the kernel that walks pages without LDS
# staging), and one that is no multiple of 4 either (the float32-arithmetic kernel takes it, whatever the storage
# type); then head sizes above 256 (the general kernel with a larger tile) and one that is no multiple of 16
ATT_SHAPES = [(4, 2, 16, 16), (3, 1, 32, 8), (5, 5, 48, 16), (14, 2, 64, 16), (8, 2, 128, 32), (6, 3, 80, 4), (2, 1, 256, 16),
              (4, 2, 64, 12), (5, 1, 48, 6), (2, 1, 320, 16), (1, 1, 512, 8), (3, 1, 40, 16)]
ATT_BATCHES = [[(1, 1)], [(17, 17)], [(70, 1), (33, 33), (9, 2), (130, 5)], [(300, 300)], [(513, 1), (64, 64), (257, 2)]]


@pytest.mark.parametrize("nq,nkv,hd,page", ATT_SHAPES)
@pytest.mark.parametrize("batch", range(len(ATT_BATCHES)))
@pytest.mark.parametrize("dtype,kind", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 0)])
def test_attention_mixed_batches(nq, nkv, hd, page, batch, dtype, kind):
    got, want = run_attention(dtype, nq, nkv, hd, page, ATT_BATCHES[batch], kind=kind, seed=batch)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert not np.isnan(got).any()
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,hd,page", [(4, 2, 64, 16), (14, 2, 64, 16), (16, 1, 32, 8), (5, 5, 48, 16), (20, 1, 16, 4),
                                            (6, 3, 80, 12)])
@pytest.mark.parametrize("window", [None, 300])
def test_attention_one_query_each_on_the_float32_kernel(dtype, nq, nkv, hd, page, window):
    """A step in which every sequence brings one query: the float32-arithmetic kernel then takes the query heads of
    a key/value head as the rows of a block (groups of 2 to 16; one head a group and groups of 20 go the other way),
    with the keys of long contexts shared out in chunks and joined.  One far key of the second sequence stands out."""
    seqs = [(700, 1), (2049, 1), (33, 1), (1, 1), (512, 1), (257, 1)]
    got, want = run_attention(dtype, nq, nkv, hd, page, seqs, window=window, kind=1, spike=(1, 1800), seed=nq)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert not np.isnan(got).any()
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("dtype,kind", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 0)])
@pytest.mark.parametrize("nq,nkv,hd,page", [(14, 2, 64, 16), (16, 1, 32, 8), (6, 3, 80, 12), (4, 4, 48, 4)])
def test_attention_never_reads_past_a_sequence_s_table_row(dtype, kind, nq, nkv, hd, page):
    """One-query sequences whose contexts fill the last page of their table row, the rows no wider than that: the
    entry after a row's end is the next sequence's first page, here full of NaN.  A kernel that walks even one key
    past its context multiplies that NaN by a zero probability and spoils the row."""
    ctx = 8 * page
    seqs = [(ctx, 1), (3, 1), (ctx, 1), (ctx - 1, 1), (5, 1)]
    got, want = run_attention(dtype, nq, nkv, hd, page, seqs, kind=kind, seed=hd, exact_table=True, poison=1)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    keep = [0, 2, 3, 4]
    assert not np.isnan(got[keep]).any()           # the poisoned sequence's own row may hold anything
    assert np.abs(got[keep] - want[keep]).max() <= tol * (1 + np.abs(want[keep]).max())


@pytest.mark.parametrize("dtype,kind", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 0)])
@pytest.mark.parametrize("window", [1, 5, 16, 33, 100])
def test_attention_window_edges(dtype, kind, window):
    got, want = run_attention(dtype, 4, 2, 32, 8, [(90, 1), (90, 40), (7, 7), (200, 3)], window=window, kind=kind, seed=window)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("dtype,kind", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 0)])
@pytest.mark.parametrize("far", [0, 15, 16, 255, 256, 640, 699])
def test_attention_finds_one_far_key_among_hundreds(dtype, kind, far):
    """One key's score dominates; the output of the last query is that key's value row."""
    got, want = run_attention(dtype, 4, 2, 64, 16, [(700, 1), (700, 9)], kind=kind, spike=(1, far), seed=far)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("dtype,kind", [(torch.float32, 1), (torch.bfloat16, 0)])
@pytest.mark.parametrize("nq,nkv,hd,page", [(4, 2, 64, 16), (3, 1, 32, 8), (6, 3, 80, 32), (8, 2, 128, 16)])
@pytest.mark.parametrize("window", [None, 300])
def test_attention_few_queries_over_a_long_context(dtype, kind, nq, nkv, hd, page, window):
    """A portion of a long prompt beside short sequences: few tiles with a long walk over the keys, which
    the bfloat16 kernel shares out between several blocks per tile and merges afterwards."""
    seqs = [(3000, 40), (90, 90), (700, 1), (1537, 17), (129, 2)]
    got, want = run_attention(dtype, nq, nkv, hd, page, seqs, window=window, kind=kind, seed=hd)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert not np.isnan(got).any()
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("nq,nkv,hd,page", [(8, 8, 32, 8), (16, 8, 32, 16), (14, 2, 64, 16), (24, 8, 80, 32)])
@pytest.mark.parametrize("seqs,window", [([(2080, 2080)], None), ([(1500, 1000), (1100, 1100), (40, 40)], None),
                                         ([(1500, 1000), (1100, 1100), (40, 40)], 300)])
def test_attention_long_prompts_whose_tiles_are_taken_in_pairs(nq, nkv, hd, page, seqs, window):
    """Enough tiles that the bfloat16 prefill kernel gives each block a long walk and a short one (an odd
    number of tiles: the middle one is taken once), with one, two, four and three query heads per group."""
    got, want = run_attention(torch.bfloat16, nq, nkv, hd, page, seqs, window=window, kind=0, seed=nq)
    assert not np.isnan(got).any()
    assert np.abs(got - want).max() <= 2e-2 * (1 + np.abs(want).max())


@pytest.mark.parametrize("dtype,kind", [(torch.bfloat16, 0), (torch.float32, 1)])
@pytest.mark.parametrize("far", [0, 127, 128, 255, 256, 511, 512, 1000, 2047, 2999])
def test_attention_split_walk_finds_one_far_key(far, dtype, kind):
    """Both kernels share the keys of these few tiles out over several blocks (the float32 one in chunks of 256)."""
    got, want = run_attention(dtype, 4, 2, 64, 16, [(3000, 1), (3000, 9)], kind=kind, spike=(1, far), seed=far)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("nq,nkv,hd,page", [(14, 2, 64, 16), (8, 2, 128, 16), (3, 1, 32, 8)])
@pytest.mark.parametrize("window", [None, 5000])
@pytest.mark.parametrize("dtype,kind", [(torch.bfloat16, 0), (torch.float32, 1)])
def test_attention_decodes_over_long_contexts(nq, nkv, hd, page, window, dtype, kind):
    """One query each over thousands of keys: more chunks than one wave of the merge kernel takes in a trip
    (several waves share them, unevenly), beside a short sequence whose chunks are nearly all empty.  The
    float32 kernel shares the keys out in 32 chunks of 640."""
    seqs = [(9000, 1), (100, 1), (20000, 1), (4097, 1)]
    got, want = run_attention(dtype, nq, nkv, hd, page, seqs, window=window, kind=kind, seed=hd)
    assert not np.isnan(got).any()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("nq,nkv,hd,page,hidden", [(14, 2, 64, 16, 896), (3, 1, 32, 8, 100), (4, 4, 128, 16, 264),
                                                   (5, 1, 96, 4, 17), (6, 2, 48, 16, 1000), (2, 1, 16, 32, 64)])
@pytest.mark.parametrize("contexts", [[300], [257, 4096, 1000, 513, 300, 2049, 777, 4000], list(range(258, 258 + 40 * 20, 20)),
                                      [1, 5000, 256, 255], [4096 - 61 * i for i in range(64)], [4096 - 120 * i for i in range(32)],
                                      list(range(300, 300 + 17 * 200, 200)), list(range(258, 258 + 25 * 150, 150))])
@pytest.mark.parametrize("window", [None, 700])
def test_attention_decode_with_the_projection_folded_in(nq, nkv, hd, page, hidden, contexts, window):
    """Decoded tokens only, contexts of several chunks of keys: the merge of the chunks multiplies by the
    output projection and adds into the residual.  1, 8, 4, 32, 17 and 25 sequences (one or two tiles of 16
    sequences, the last one full, partly filled or holding a single sequence; with more than 16 sequences a block
    takes one or two tiles of rows a wave, by the number of heads and the width), among them contexts of a
    single chunk and of one key, whose other chunks are empty; 40 and 64 sequences are declined."""
    got, want = run_attention(torch.bfloat16, nq, nkv, hd, page, [(c, 1) for c in contexts], window=window, kind=0,
                              seed=hidden, hidden=hidden)
    assert not np.isnan(got).any()
    assert np.abs(got - want).max() <= 2e-2 * (1 + np.abs(want).max())


@pytest.mark.parametrize("far", [0, 4095, 4096, 12345, 19999])
def test_attention_decode_finds_one_far_key_among_thousands(far):
    got, want = run_attention(torch.bfloat16, 4, 2, 64, 16, [(300, 1), (20000, 1)], kind=0, spike=(1, far), seed=far)
    assert np.abs(got - want).max() <= 2e-2 * (1 + np.abs(want).max())


def test_attention_refuses_what_it_cannot_take():
    from sprout_lm_amd import ops
    q = torch.zeros(1, 4 * 16, device=DEV)
    pool = torch.zeros(2, 3, 16, 16, device=DEV)
    batch = ops.AttentionBatch.build([1], [1], DEV)
    table = torch.zeros(1, 2, dtype=torch.int32, device=DEV)
    with pytest.raises(ops.KernelError, match="groups"):
        ops.attention(q, 64, pool, pool, table, batch, torch.empty_like(q), 4, 3, 16, None, 0.25, kind=1)
    big = torch.zeros(1, 528, device=DEV)
    pool = torch.zeros(2, 1, 16, 528, device=DEV)
    with pytest.raises(ops.KernelError, match="head size 528 is outside 1..512"):
        ops.attention(big, 528, pool, pool.transpose(2, 3).contiguous(), table, batch, torch.empty_like(big), 1, 1, 528, None, 0.1, kind=1)


@pytest.mark.parametrize("dtype,kind", [(torch.bfloat16, 0), (torch.float32, 1)])
@pytest.mark.parametrize("seqs", [[(300, 1), (1, 1), (257, 1), (520, 1), (33, 1)], [(200, 200)], [(330, 70), (40, 1), (64, 64)]])
def test_attention_at_the_head_counts_of_the_largest_model(dtype, kind, seqs):
    """40 query heads in 8 groups of head size 128 (the 32B sizes): decoded tokens, a whole prompt, a mixed step."""
    got, want = run_attention(dtype, 40, 8, 128, 16, seqs, kind=kind, seed=len(seqs))
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert not np.isnan(got).any()
    assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max())


@pytest.mark.parametrize("T", [1, 8, 40, 300])
@pytest.mark.parametrize("what", ["down", "gate_up", "qkv", "head"])
def test_products_at_the_widths_of_the_largest_model(T, what):
    """The products of the 32B sizes (a width of 5,120, 27,648 inner columns, 40 + 8 + 8 heads of 128) against a
    float32 product of the same bfloat16 operands: every kernel that generation takes at these widths."""
    from sprout_lm_amd import ops
    gen = torch.Generator(device=DEV).manual_seed(T)
    H, I, V = 5120, 27648, 152064
    rand = lambda *shape, scale=1.0: (torch.randn(*shape, device=DEV, generator=gen) * scale).to(torch.bfloat16)
    if what == "down":
        x, w = rand(T, I), rand(H, I, scale=I ** -0.5)
        before = torch.randn(T, H, device=DEV, generator=gen)
        out = before.clone()
        ops.gemm(x, w, out, accumulate=True)
        want = before + x.float() @ w.float().T
        tol = 2e-3          # float32 sums of 27,648 products, in another order
    elif what == "gate_up":
        x, w = rand(T, H), rand(2 * I, H, scale=H ** -0.5)
        out = torch.empty(T, I, dtype=torch.bfloat16, device=DEV)
        ops.gate_up_silu(w, out, x=x)
        gu = (x.float() @ w.float().T).to(torch.bfloat16).float()
        want = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
        out, tol = out.float(), 2 ** -6
    elif what == "qkv":
        N = (40 + 2 * 8) * 128
        x, w, b = rand(T, H), rand(N, H, scale=H ** -0.5), rand(N, scale=0.3)
        out = torch.empty(T, N, dtype=torch.bfloat16, device=DEV)
        ops.gemm(x, w, out, bias=b)
        want = x.float() @ w.float().T + b.float()
        out, tol = out.float(), 2 ** -7
    else:
        T = min(T, 64)          # logits are asked for at a few places
        x, w = rand(T, H), rand(V, H, scale=H ** -0.5)
        out = torch.empty(T, V, dtype=torch.float32, device=DEV)
        ops.gemm(x, w, out)
        want = x.float() @ w.float().T
        tol = 2e-3
    err = (out - want).abs().max().item()
    assert err <= tol * (1 + want.abs().max().item()), f"{what} at {T} tokens: {err:.3e}"


def test_variants_without_a_kernel_are_refused_by_the_library_itself():
    """A rotation's pairing and a gate's activation are parameters of the C entry points; a value that no
    kernel implements comes back as an error, whoever calls."""
    from sprout_lm_amd import ops
    lib = ops.library()
    stream = torch.cuda.current_stream().cuda_stream
    qkv = torch.zeros(2, 4 * 16, device=DEV)
    pos = torch.zeros(2, dtype=torch.int32, device=DEV)
    inv = torch.ones(8, device=DEV)
    args = (stream, 0, qkv.data_ptr(), pos.data_ptr(), inv.data_ptr(), None, 16, None, None, None, 2, 4, 0, 16, 0, 0)
    assert lib.sp_rope_cache(*args, 0) == 0
    assert lib.sp_rope_cache(*args, 1) != 0 and b"pairing 1" in lib.sp_last_error()
    gu = torch.zeros(2, 32, device=DEV)
    out = torch.zeros(2, 16, device=DEV)
    assert lib.sp_silu_mul(stream, 0, gu.data_ptr(), out.data_ptr(), 2, 16, 0) == 0
    assert lib.sp_silu_mul(stream, 0, gu.data_ptr(), out.data_ptr(), 2, 16, 3) != 0 and b"activation 3" in lib.sp_last_error()
    assert lib.sp_fused_supported(ops.FUSED_ROPE, 8, 1152, 896, 64, 64, 0, 0) == 1
    assert lib.sp_fused_supported(ops.FUSED_ROPE, 8, 1152, 896, 64, 64, 0, 1) == 0
    assert lib.sp_fused_supported(ops.FUSED_SILU, 8, 9728, 896, 0, 0, 0, 2) == 0
    assert not ops.fused_supported(ops.FUSED_SILU, 8, 9728, 896, variant="gelu")
    with pytest.raises(ops.KernelError, match="activation 'relu'"):
        ops.silu_mul(gu, out, activation="relu")
    # what stands between q . k and the softmax is such a parameter of the attention entry points
    q = torch.zeros(1, 32, device=DEV)
    kp, vp = torch.zeros(2, 1, 8, 16, device=DEV), torch.zeros(2, 1, 16, 8, device=DEV)
    batch = ops.AttentionBatch.build([1], [1], DEV)
    tables = torch.zeros(1, 1, dtype=torch.int32, device=DEV)
    assert ops.attention(q, 32, kp, vp, tables, batch, torch.zeros_like(q), 2, 1, 16, None, 0.25) is False
    with pytest.raises(ops.KernelError, match="score stage 'soft_cap'"):
        ops.attention(q, 32, kp, vp, tables, batch, torch.zeros_like(q), 2, 1, 16, None, 0.25, scores="soft_cap")
    torch.cuda.synchronize()


def test_sampling_greedy_ties_nonfinite_and_temperature():
    from sprout_lm_amd import ops
    V = 151936 // 8 + 13
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((5, V)).astype(np.float32)
    logits[1, [70, 9000, 18000]] = 9.0                      # ties: the lowest index wins
    logits[2, 555] = np.nan
    logits[3, V - 1] = 50.0
    logits[4, 17] = np.inf
    L = t(logits)
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    ws = torch.empty(ops.sample_workspace_floats(5, V), device=DEV)
    ops.sample(L, out, ws)
    assert out.tolist() == [int(np.argmax(logits[0])), 70, -1, V - 1, -1]
    # temperature: reproducible, keyed by (seed, counter), and distributed as softmax(logits / T)
    small = np.log(np.array([[0.5, 0.25, 0.125, 0.125]], np.float32)).repeat(4000, 0)
    S = t(small)
    temp = torch.full((4000,), 1.0, device=DEV)
    seed = torch.full((4000,), 42, dtype=torch.int64, device=DEV)
    counter = torch.arange(4000, dtype=torch.int32, device=DEV)
    out = torch.empty(4000, dtype=torch.int32, device=DEV)
    ws = torch.empty(ops.sample_workspace_floats(4000, 4), device=DEV)
    ops.sample(S, out, ws, temp, seed, counter)
    first = out.clone()
    ops.sample(S, out, ws, temp, seed, counter)
    assert torch.equal(first, out)
    freq = np.bincount(first.cpu().numpy(), minlength=4) / 4000
    assert np.abs(freq - [0.5, 0.25, 0.125, 0.125]).max() < 0.03
    ops.sample(S, out, ws, temp, seed + 1, counter)
    assert not torch.equal(first, out)
    # row r of a batch draws what it would draw alone
    ops.sample(S[10:11].contiguous(), out[:1], ws, temp[:1], seed[:1], counter[10:11].contiguous())
    assert out[0].item() == first[10].item()
    cold = torch.full((4000,), 0.05, device=DEV)
    ops.sample(S, out, ws, cold, seed, counter)
    assert (out == 0).float().mean().item() > 0.99


@pytest.mark.parametrize("hd,rotary,theta", [(48, 48, 50000.0), (64, 64, 1e6), (32, 16, 10000.0)])
def test_rope_with_float64_angles_at_far_positions(hd, rotary, theta):
    """Float32 storage with the tail of the frequency table: angles are exact to float64 rounding, so positions
    in the tens of thousands turn as exactly as position 1 (a float32 angle would be off by 1e-3 there)."""
    from sprout_lm_amd import ops
    rng = np.random.default_rng(hd)
    T, nq = 9, 3
    x = rng.standard_normal((T, nq * hd)).astype(np.float32)
    pos = np.array([0, 1, 999, 4097, 12345, 20000, 31999, 32767, 100000])
    exact = theta ** (-2.0 * np.arange(rotary // 2) / rotary)
    head = torch.tensor(exact, dtype=torch.float32)
    tail = torch.tensor(exact - head.double().numpy(), dtype=torch.float32)
    with_tail, without = t(x), t(x)
    ops.rope_cache(with_tail, torch.tensor(pos, dtype=torch.int32, device=DEV), head.to(DEV), rotary, nq, 0, hd,
                   inv_freq_tail=tail.to(DEV))
    ops.rope_cache(without, torch.tensor(pos, dtype=torch.int32, device=DEV), head.to(DEV), rotary, nq, 0, hd)
    want = plain_rope(x, pos, hd, rotary, theta)
    assert np.abs(with_tail.cpu().numpy() - want).max() <= 1e-6
    assert np.abs(without.cpu().numpy() - want).max() > 1e-5    # what the tail is for


# ---- decode-sized fused kernels --------------------------------------------------------------------

def _normed(res, w, eps):
    x = res.astype(np.float64)
    return bf16(x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w)


@pytest.mark.parametrize("T", [1, 3, 16, 17, 40, 64, 65, 200, 513])   # above 64: the tiled product's rotating epilogue
# (4, 2, 128, 3584) and (3, 1, 64, 2120): few rows with a long K (a block asks for twice the steps at once); (28, 4, 128,
# 512): more rotation pairs than 256 blocks of 8 hold, so a block takes 9 of them in two tiles, across the heads' ends;
# (14, 2, 64, 896): 3 pairs a block, which 32 pairs a head do not divide
@pytest.mark.parametrize("nq,nkv,hd,K,page", [(14, 2, 64, 896, 16), (3, 1, 32, 96, 8), (4, 4, 128, 264, 16), (5, 1, 96, 240, 4),
                                              (4, 2, 128, 3584, 16), (3, 1, 64, 2120, 8), (4, 2, 16, 64, 16), (5, 5, 48, 240, 16),
                                              (2, 1, 80, 160, 4), (5, 1, 64, 320, 8), (3, 3, 128, 384, 16), (28, 4, 128, 512, 16)])
@pytest.mark.parametrize("norm", [False, True])
def test_fused_qkv_rope_cache(T, nq, nkv, hd, K, page, norm):
    check_fused_qkv_rope_cache(T, nq, nkv, hd, K, page, norm)


# The rotating epilogue on each block shape that takes it: (T, nq, nkv, hd, K) -> (block rows, block columns, waves).
# The plan is asserted: a size that has moved to another shape says so.
ROTATING_SHAPE_SIZES = {
    (200, 28, 4, 128, 896): (64, 128, 4), (264, 28, 4, 128, 3584): (64, 128, 4), (1024, 14, 2, 64, 896): (64, 128, 4),
    (400, 28, 4, 128, 448): (128, 128, 8), (513, 28, 4, 128, 3584): (128, 128, 8), (2048, 14, 2, 64, 896): (128, 128, 8),
    (1024, 28, 4, 128, 448): (256, 128, 8), (1024, 28, 4, 128, 896): (256, 128, 8),
}


@pytest.mark.parametrize("case", sorted(ROTATING_SHAPE_SIZES))
def test_fused_qkv_rope_cache_on_every_block_shape(case):
    from sprout_lm_amd import ops
    T, nq, nkv, hd, K = case
    rows, cols, splits, waves = ops.pipe_plan(ops.PLAN_ROTATING, T, (nq + 2 * nkv) * hd, K, hd)
    assert (rows, cols, waves) == ROTATING_SHAPE_SIZES[case] and splits == 1, "this size has moved to another block shape"
    check_fused_qkv_rope_cache(T, nq, nkv, hd, K, 16, False)


def check_fused_qkv_rope_cache(T, nq, nkv, hd, K, page, norm):
    from sprout_lm_amd import ops
    taken = ops.fused_supported(ops.FUSED_ROPE, T, (nq + 2 * nkv) * hd, K, hd, hd, norm)
    rng = np.random.default_rng(T * 7 + hd)
    N, pages, theta, eps = (nq + 2 * nkv) * hd, max(40, -(-T // page) + 1), 10000.0, 1e-5
    w = bf16(rng.standard_normal((N, K)) / math.sqrt(K))
    b = bf16(rng.standard_normal(N) * 0.3)
    res = (rng.standard_normal((T, K)) * 2).astype(np.float32)
    nw = bf16(rng.uniform(0.5, 1.5, K))
    x = _normed(res, nw, eps) if norm else bf16(res)
    pos = rng.integers(0, 300, T)
    slots = rng.permutation(pages * page)[:T].astype(np.int32)
    if T > 2:
        slots[2] = -1
    inv = torch.tensor(theta ** (-2.0 * np.arange(hd // 2) / hd), dtype=torch.float32, device=DEV)
    kp = torch.zeros(pages, nkv, page, hd, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(pages, nkv, hd, page, dtype=torch.bfloat16, device=DEV)
    q_out = torch.full((T, nq * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    args = dict(residual=t(res), norm_weight=t(nw, torch.bfloat16), eps=eps) if norm else dict(x=t(x, torch.bfloat16))
    call = lambda: ops.qkv_rope_cache(t(w, torch.bfloat16), t(b, torch.bfloat16), q_out, t(pos, torch.int32), inv, hd,
                                      t(slots, torch.int32), kp, vp, nq, nkv, hd, **args)
    if not taken:       # a shape the kernel does not take is refused, never computed wrongly
        with pytest.raises(ops.KernelError):
            call()
        return
    call()
    qkv = bf16(x.astype(np.float64) @ w.astype(np.float64).T + b)
    want = plain_rope(qkv[:, :(nq + nkv) * hd], pos, hd, hd, theta)
    got_q = q_out.float().cpu().numpy()
    scale = 1 + np.abs(want).max()
    assert np.abs(got_q - want[:, :nq * hd]).max() <= 2 ** -7 * scale
    kp, vp = kp.float().cpu().numpy(), vp.float().cpu().numpy().transpose(0, 1, 3, 2)
    for i in range(T):
        if slots[i] < 0:
            continue
        pg, off = divmod(int(slots[i]), page)
        assert np.abs(kp[pg, :, off].reshape(-1) - want[i, nq * hd:]).max() <= 2 ** -7 * scale
        assert np.abs(vp[pg, :, off].reshape(-1) - qkv[i, (nq + nkv) * hd:]).max() <= 2 ** -7 * scale
    written = np.zeros((pages, page), bool)
    written[[s // page for s in slots if s >= 0], [s % page for s in slots if s >= 0]] = True
    assert np.all((kp == 0) | written[:, None, :, None]) and np.all((vp == 0) | written[:, None, :, None])
    if T > 64:   # with the step's table of cosines and sines the result is the same to the bit
        table = torch.empty(T, hd // 2, 2, dtype=torch.float32, device=DEV)
        ops.rope_table(t(pos, torch.int32), inv, table)
        angles = pos[:, None].astype(np.float32) * inv.cpu().numpy()[None, :]
        assert np.abs(table.cpu().numpy() - np.stack([np.cos(angles.astype(np.float64)), np.sin(angles.astype(np.float64))], -1)).max() < 1e-6
        kp2, vp2, q2 = torch.zeros_like(t(kp, torch.bfloat16)), torch.zeros_like(t(vp, torch.bfloat16)), torch.zeros_like(q_out)
        vp2 = torch.zeros(pages, nkv, hd, page, dtype=torch.bfloat16, device=DEV)
        ops.qkv_rope_cache(t(w, torch.bfloat16), t(b, torch.bfloat16), q2, t(pos, torch.int32), inv, hd,
                           t(slots, torch.int32), kp2, vp2, nq, nkv, hd, table=table, **args)
        assert torch.equal(q2, q_out)
        assert np.array_equal(kp2.float().cpu().numpy(), kp) and np.array_equal(vp2.float().cpu().numpy().transpose(0, 1, 3, 2), vp)


@pytest.mark.parametrize("T,I,K", [(t_, i_, k_) for t_ in [1, 8, 16, 33, 64, 65, 200, 513]
                                   for i_, k_ in [(4864, 896), (224, 96), (176, 240), (1000, 264), (331, 72), (160, 2312)]]
                         + [(1100, 6700, 128), (2048, 4864, 896),   # blocks of 384 tokens
                            (1024, 2432, 264), (200, 1000, 3584),   # blocks of 256 x 128 and 128 x 128 on eight waves
                            (513, 18944, 896), (130, 9472, 448), (264, 18944, 448)])  # blocks of 256 x 256, of 64 x 128, one of 384
@pytest.mark.parametrize("norm", [False, True])
def test_fused_gate_up_silu_and_normed_product(T, I, K, norm):
    from sprout_lm_amd import ops
    taken = ops.fused_supported(ops.FUSED_SILU, T, 2 * I, K, norm=norm)
    rng = np.random.default_rng(T + I)
    eps = 1e-6
    w = bf16(rng.standard_normal((2 * I, K)) / math.sqrt(K) * 2)
    res = (rng.standard_normal((T, K)) * 3).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, K).astype(np.float32)       # a norm weight kept in 32-bit
    x = _normed(res, nw, eps) if norm else bf16(res)
    args = dict(residual=t(res), norm_weight=t(nw), eps=eps) if norm else dict(x=t(x, torch.bfloat16))
    out = torch.empty(T, I, dtype=torch.bfloat16, device=DEV)
    if not taken:
        with pytest.raises(ops.KernelError):
            ops.gate_up_silu(t(w, torch.bfloat16), out, **args)
        return
    ops.gate_up_silu(t(w, torch.bfloat16), out, **args)
    gu = bf16(x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float64)
    g, u = gu[:, :I], gu[:, I:]
    want = g / (1 + np.exp(-g)) * u
    assert np.abs(out.float().cpu().numpy() - want).max() <= 2 ** -6 * (1 + np.abs(want).max())


@pytest.mark.parametrize("T", [1, 8, 16])
@pytest.mark.parametrize("nq,nkv,hd,K,page", [(14, 2, 64, 896, 16), (3, 1, 32, 96, 8), (4, 4, 128, 264, 16), (2, 1, 96, 64, 4),
                                              (4, 2, 16, 64, 16), (5, 5, 48, 240, 16), (2, 1, 32, 2116, 8)])
@pytest.mark.parametrize("norm", [False, True])
def test_float32_qkv_with_norm_rotation_and_cache_write_folded_in(T, nq, nkv, hd, K, page, norm):
    """The float32 path's q/k/v product of a decode step: bias, rotation with float64 angles at far positions and
    the cache write in its epilogue, the norm before it as its prologue; against float64 arithmetic."""
    from sprout_lm_amd import ops
    rng = np.random.default_rng(T * 11 + hd)
    N, pages, theta, eps = (nq + 2 * nkv) * hd, 40, 1e6, 1e-5
    w = (rng.standard_normal((N, K)) / math.sqrt(K)).astype(np.float32)
    b = (rng.standard_normal(N) * 0.3).astype(np.float32)
    res = (rng.standard_normal((T, K)) * 2).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, K).astype(np.float32)
    x = res.astype(np.float64)
    if norm:
        x = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * nw
    pos = rng.integers(0, 30000, T)
    slots = rng.permutation(pages * page)[:T].astype(np.int32)
    if T > 2:
        slots[2] = -1
    exact = theta ** (-2.0 * np.arange(hd // 2) / hd)
    inv = torch.tensor(exact, dtype=torch.float32, device=DEV)
    tail = torch.tensor(exact - inv.cpu().double().numpy(), dtype=torch.float32, device=DEV)
    kp = torch.zeros(pages, nkv, page, hd, device=DEV)
    vp = torch.zeros(pages, nkv, hd, page, device=DEV)
    q_out = torch.full((T, nq * hd), float("nan"), device=DEV)
    assert ops.qkv_rope_cache_f32(t(w), t(b), t(res), q_out, t(pos, torch.int32), inv, tail, hd, t(slots, torch.int32), kp, vp,
                                  nq, nkv, hd, norm_weight=t(nw) if norm else None, eps=eps)
    qkv = x @ w.astype(np.float64).T + b
    want = plain_rope(qkv[:, :(nq + nkv) * hd], pos, hd, hd, theta)
    tol = 1e-5 * max(1, math.sqrt(K) / 8) * (1 + np.abs(qkv).max())
    assert np.abs(q_out.cpu().numpy() - want[:, :nq * hd]).max() <= tol
    kp, vp = kp.cpu().numpy(), vp.cpu().numpy().transpose(0, 1, 3, 2)
    for i in range(T):
        if slots[i] < 0:
            continue
        pg, off = divmod(int(slots[i]), page)
        assert np.abs(kp[pg, :, off].reshape(-1) - want[i, nq * hd:]).max() <= tol
        assert np.abs(vp[pg, :, off].reshape(-1) - qkv[i, (nq + nkv) * hd:]).max() <= tol
    written = np.zeros((pages, page), bool)
    written[[s // page for s in slots if s >= 0], [s % page for s in slots if s >= 0]] = True
    assert np.all((kp == 0) | written[:, None, :, None]) and np.all((vp == 0) | written[:, None, :, None])
    # shapes it does not take are declined, nothing is written
    assert not ops.qkv_rope_cache_f32(t(w[:(nq + 2 * nkv) * 24]), None, t(res), torch.empty(T, nq * 24, device=DEV),
                                      t(pos, torch.int32), inv, None, 24, t(slots, torch.int32),
                                      torch.zeros(pages, nkv, page, 24, device=DEV), torch.zeros(pages, nkv, 24, page, device=DEV),
                                      nq, nkv, 24)


@pytest.mark.parametrize("T,I,K", [(8, 4864, 896), (16, 37, 132), (3, 100, 4864)])
def test_gated_product_of_few_tokens_in_float32_with_the_norm_folded_in(T, I, K):
    from sprout_lm_amd import ops
    rng = np.random.default_rng(T + I + K + 1)
    res = (rng.standard_normal((T, K)) * 3).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, K).astype(np.float32)
    w = (rng.standard_normal((2 * I, K)) * 2 / math.sqrt(K)).astype(np.float32)
    x = res.astype(np.float64)
    x = x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6) * nw
    gate, up = x @ w[:I].astype(np.float64).T, x @ w[I:].astype(np.float64).T
    want = gate / (1 + np.exp(-gate)) * up
    out = torch.full((T, I), float("nan"), dtype=torch.float32, device=DEV)
    assert ops.gate_up_silu_f32(t(w), t(res), out, norm_weight=t(nw), eps=1e-6)
    assert np.abs(out.cpu().numpy() - want).max() <= 1e-5 * max(1, math.sqrt(K) / 8) * (1 + np.abs(want).max())
