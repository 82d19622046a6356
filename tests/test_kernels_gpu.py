"""Each HIP kernel alone against its plain PyTorch reference (tests/emu_ops.py), at sizes other
than the engine's: widths and vocabularies that are no power of two, odd head counts and groups,
head sizes in steps of 16 and below, ragged batches, shuffled pages."""
import math

import pytest
import torch

from emu_ops import EmuOps

pytestmark = pytest.mark.gpu
emu = EmuOps()
DEV = "cuda:0"


def _ops():
    from tempura_amd.kernels import ops
    ops.set_backend(None)
    return ops


def _close(got, ref, tol, what=""):
    err = float((got.double().cpu() - ref.double()).abs().max())
    scale = float(ref.double().abs().max()) or 1.0
    assert err <= tol * scale, f"{what}: max error {err:.3e} against scale {scale:.3e} (tol {tol})"


def _tol(dtype):
    return 1e-5 if dtype == torch.float32 else 1.2e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,hidden,vocab", [(1, 64, 256), (7, 100, 301), (33, 4096, 1000)])
def test_embed(dtype, n, hidden, vocab):
    ops = _ops()
    g = torch.Generator().manual_seed(1)
    table = torch.randn(vocab, hidden, generator=g).to(dtype)
    tok = torch.randint(0, vocab, (n,), generator=g, dtype=torch.int32)
    got = ops.embed(tok.to(DEV), table.to(DEV))
    assert torch.equal(got.cpu(), emu.embed(tok, table))


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,hidden,eps", [(1, 16, 1e-5), (4, 64, 1e-6), (8, 256, 1e-5), (3, 100, 1e-2), (5, 4096, 1e-5), (2, 5000, 1e-6)])
def test_rmsnorm(out_dtype, n, hidden, eps):
    ops = _ops()
    g = torch.Generator().manual_seed(2)
    x = torch.randn(n, hidden, generator=g) * 3
    x[0] *= 1e-3                                  # a near-zero row: eps placement matters
    w = 1 + 0.3 * torch.randn(hidden, generator=g)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, out_dtype)
    _close(got, emu.rmsnorm(x, w, eps, torch.float64), _tol(out_dtype), "rmsnorm")
    rows = torch.tensor([n - 1, 0], dtype=torch.int32)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, out_dtype, rows.to(DEV))
    _close(got, emu.rmsnorm(x, w, eps, torch.float64, rows), _tol(out_dtype), "rmsnorm rows")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1, 16, 8), (4, 32, 16), (8, 64, 64), (1, 1024, 512), (3, 96, 320), (9, 12, 96),
                                   (17, 100, 36), (64, 384, 96), (65, 130, 70), (130, 257, 129), (2, 301, 1000)])
def test_linear(dtype, m, n, k):
    ops = _ops()
    g = torch.Generator().manual_seed(3)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = torch.randn(n, k, generator=g).to(dtype)
    ref = x.double() @ w.double().T
    for out_dtype in ([torch.float32] if dtype == torch.float32 else [torch.float32, torch.bfloat16]):
        got = ops.linear(x.to(DEV), w.to(DEV), out_dtype)
        _close(got, ref, 1e-5 if out_dtype == torch.float32 else 1e-2, f"linear {out_dtype}")
    res = torch.randn(m, n, generator=g)
    got = ops.linear(x.to(DEV), w.to(DEV), torch.float32, residual=res.clone().to(DEV))
    _close(got, ref + res.double(), 1e-5, "linear residual")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,d,rot,page", [(4, 2, 16, 16, 16), (8, 1, 12, 12, 8), (6, 3, 48, 48, 32), (3, 3, 80, 32, 4), (32, 8, 128, 128, 16)])
def test_rope_kv_write(dtype, heads, kv, d, rot, page):
    ops = _ops()
    from tempura_amd.parts.rope import rotary_inv_freq
    g = torch.Generator().manual_seed(4)
    n, pages = 19, 7
    qkv = torch.randn(n, (heads + 2 * kv) * d, generator=g)
    pos = torch.randint(0, 100000, (n,), generator=g, dtype=torch.int32)
    slots = torch.randperm(pages * page, generator=g)[:n].to(torch.int32)
    inv = rotary_inv_freq(d, 500000.0, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                        "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}, rot)
    kc = torch.zeros(pages, kv, page, d, dtype=dtype)
    vc = torch.zeros(pages, kv, d, page, dtype=dtype)
    kr, vr = kc.clone(), vc.clone()
    qr = emu.rope_kv_write(qkv, pos, slots, inv, rot, 1.0, heads, kv, d, kr, vr, torch.float64)
    kd, vd = kc.to(DEV), vc.to(DEV)
    q = ops.rope_kv_write(qkv.to(DEV), pos.to(DEV), slots.to(DEV), inv.to(DEV), rot, 1.0, heads, kv, d, kd, vd, dtype)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    _close(q, qr, tol, "q")
    _close(kd, kr, tol, "k cache")
    _close(vd, vr, tol, "v cache")
    # queries only (a call that reads another call's cache)
    q2 = ops.rope_kv_write(qkv[:, : heads * d].contiguous().to(DEV), pos.to(DEV), None, inv.to(DEV), rot, 1.0,
                           heads, kv, d, None, None, dtype)
    assert torch.equal(q2, q)
    # cosines and sines from the step's table: the same bits as when the kernel computes them itself
    if rot:
        table = ops.rope_table(pos.to(DEV), inv.to(DEV), rot, 1.0)
        k3, v3 = kc.to(DEV), vc.to(DEV)
        q3 = ops.rope_kv_write(qkv.to(DEV), pos.to(DEV), slots.to(DEV), inv.to(DEV), rot, 1.0, heads, kv, d, k3, v3,
                               dtype, table)
        assert torch.equal(q3, q) and torch.equal(k3, kd) and torch.equal(v3, vd)
        ang = pos.double()[:, None] * inv.double()[None, :]
        _close(table[..., 0], torch.cos(ang), 2e-6, "table cosines")
        _close(table[..., 1], torch.sin(ang), 2e-6, "table sines")


@pytest.mark.parametrize("m,heads,kv,d,rot,k,page", [(1, 4, 2, 64, 64, 256, 16), (8, 32, 8, 128, 128, 4096, 16),
                                                    (16, 3, 1, 48, 32, 96, 8), (5, 6, 3, 16, 16, 2048, 32),
                                                    (2100, 32, 8, 128, 128, 128, 16), (3000, 24, 8, 128, 64, 192, 8),
                                                    (4300, 4, 2, 128, 128, 64, 16), (2900, 10, 1, 128, 128, 320, 16),
                                                    (520, 32, 8, 128, 128, 256, 16), (2100, 32, 8, 64, 64, 128, 16),
                                                    (3000, 5, 3, 64, 32, 192, 8), (2600, 3, 1, 192, 192, 64, 16),
                                                    (2200, 4, 2, 256, 256, 64, 16)])
def test_linear_rope_kv(m, heads, kv, d, rot, k, page):
    """The projection of a few rows that rotates and stores its rows in its epilogue gives the bits of the
    plain product followed by the rotation and cache-write kernel; and both agree with float64."""
    ops = _ops()
    from tempura_amd.parts.rope import rotary_inv_freq
    g = torch.Generator().manual_seed(7)
    n = (heads + 2 * kv) * d
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) * 0.1).to(torch.bfloat16)
    pos = torch.randint(0, 100000, (m,), generator=g, dtype=torch.int32)
    pages = 5 + (m + page - 1) // page
    if m <= 16:
        slots = torch.randperm(pages * page, generator=g)[:m].to(torch.int32)
    else:   # a portion that starts three tokens into a page and walks shuffled pages, then scattered places
        order = torch.randperm(pages, generator=g).tolist()
        first = m * 3 // 4
        sl = [order[(3 + i) // page] * page + (3 + i) % page for i in range(first)]
        used = set(sl)
        sl += [s_ for s_ in torch.randperm(pages * page, generator=g).tolist() if s_ not in used][: m - first]
        slots = torch.tensor(sl, dtype=torch.int32)
    inv = rotary_inv_freq(d, 500000.0, None, rot)
    kc = torch.zeros(pages, kv, page, d, dtype=torch.bfloat16)
    vc = torch.zeros(pages, kv, d, page, dtype=torch.bfloat16)
    xd, wd, pd, sd, invd = x.to(DEV), w.to(DEV), pos.to(DEV), slots.to(DEV), inv.to(DEV)
    k1, v1 = kc.to(DEV), vc.to(DEV)
    q1 = ops.rope_kv_write(ops.linear(xd, wd, torch.float32), pd, sd, invd, rot, 1.0, heads, kv, d, k1, v1, torch.bfloat16)
    k2, v2 = kc.to(DEV), vc.to(DEV)
    assert ops.linear_rope_ok(m, n, k, d, rot, page, torch.bfloat16, torch.bfloat16)
    q2 = ops.linear_rope_kv(xd, wd, pd, sd, invd, rot, 1.0, heads, kv, d, k2, v2,
                            ops.rope_table(pd, invd, rot, 1.0) if m > 16 else None)
    assert torch.equal(q2, q1) and torch.equal(k2, k1) and torch.equal(v2, v1)
    if rot and m <= 16:   # with the step's table of cosines and sines: the same bits again
        k3, v3 = kc.to(DEV), vc.to(DEV)
        q3 = ops.linear_rope_kv(xd, wd, pd, sd, invd, rot, 1.0, heads, kv, d, k3, v3, ops.rope_table(pd, invd, rot, 1.0))
        assert torch.equal(q3, q1) and torch.equal(k3, k1) and torch.equal(v3, v1)
    if n % 16 == 0 and k % 64 == 0:   # the weight stored tiled: the same bits
        k4, v4 = kc.to(DEV), vc.to(DEV)
        q4 = ops.linear_rope_kv(xd, ops.tile_weight(wd), pd, sd, invd, rot, 1.0, heads, kv, d, k4, v4,
                                ops.rope_table(pd, invd, rot, 1.0) if m > 16 else None)
        assert torch.equal(q4, q1) and torch.equal(k4, k1) and torch.equal(v4, v1)
    if m > 128:                        # blocks of 128 x 128 (steps of a few hundred rows): the same bits
        ops.library().tp_linear_tune_mid_tile(1)
        try:
            for wv in (wd, ops.tile_weight(wd)):
                k6, v6 = kc.to(DEV), vc.to(DEV)
                q6 = ops.linear_rope_kv(xd, wv, pd, sd, invd, rot, 1.0, heads, kv, d, k6, v6, ops.rope_table(pd, invd, rot, 1.0))
                assert torch.equal(q6, q1) and torch.equal(k6, k1) and torch.equal(v6, v1)
        finally:
            ops.library().tp_linear_tune_mid_tile(0)
    # tiles of 256 x 256 wherever the columns allow, and of 256 x 192 (whose columns span two heads of 128), asked
    # for: the same bits (with heads that such a tile's strips would cut across, the narrower tiles are taken)
    for code in ((5, 7) if m > 16 and n % 192 == 0 else (5,) if m > 16 else ()):
        ops.library().tp_linear_tune_tile(code)
        try:
            for wv in (wd, ops.tile_weight(wd)):
                k5, v5 = kc.to(DEV), vc.to(DEV)
                q5 = ops.linear_rope_kv(xd, wv, pd, sd, invd, rot, 1.0, heads, kv, d, k5, v5, ops.rope_table(pd, invd, rot, 1.0))
                assert torch.equal(q5, q1) and torch.equal(k5, k1) and torch.equal(v5, v1)
        finally:
            ops.library().tp_linear_tune_tile(0)
    kr, vr = kc.clone(), vc.clone()
    qr = emu.rope_kv_write(x.double() @ w.double().T, pos, slots, inv, rot, 1.0, heads, kv, d, kr, vr, torch.float64)
    _close(q2, qr, 1e-2, "q")
    _close(k2, kr, 1e-2, "k cache")
    _close(v2, vr, 1e-2, "v cache")


def test_rope_paired_order_is_the_split_half_rotation():
    """The kernels rotate neighbours (2 d, 2 d + 1); the reference rotates (d, d + D / 2)
    (/root/reference/kernels/src/rope.rs:18-53).  Laying a head out in paired order, rotating, and laying it
    back must give the plain implementation's split-half rotation of the same head."""
    ops = _ops()
    import plain
    g = torch.Generator().manual_seed(6)
    n, heads, d = 9, 3, 32
    half = d // 2
    x = torch.randn(n, heads, d, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 50, 777, 4095, 131071, 5], dtype=torch.int32)
    inv = plain.rope_inv_freq(d, 10000.0, None)
    want = plain.rope(x.double(), pos, inv)                      # split-half order in and out
    order = torch.arange(d)
    order[0::2] = torch.arange(half)
    order[1::2] = torch.arange(half) + half
    paired = x[:, :, order].reshape(n, heads * d).contiguous()
    got = ops.rope_kv_write(paired.to(DEV), pos.to(DEV), None, inv.to(DEV), d, 1.0, heads, 0, d, None, None, torch.float32)
    back = torch.empty_like(got.cpu())
    back[:, :, order] = got.cpu()
    _close(back, want, 2e-6, "paired rotation against the split-half formula")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,d,page,n", [(4, 2, 64, 16, 300), (3, 1, 48, 8, 277), (8, 2, 128, 32, 600), (2, 2, 12, 16, 260)])
def test_rope_kv_write_long_step(dtype, heads, kv, d, page, n):
    """Long steps store their values in runs of eight tokens where the cache places allow it: a prompt portion
    that starts in the middle of a page, single tokens scattered between, a tail that fills no run."""
    ops = _ops()
    from tempura_amd.parts.rope import rotary_inv_freq
    g = torch.Generator().manual_seed(5)
    pages = (n + page - 1) // page + 6
    qkv = torch.randn(n, (heads + 2 * kv) * d, generator=g)
    pos = torch.randint(0, 5000, (n,), generator=g, dtype=torch.int32)
    order = torch.randperm(pages, generator=g).tolist()
    first = n * 2 // 3
    # a portion of `first` tokens that starts five tokens into its first page and walks shuffled pages
    slots = [order[(5 + i) // page] * page + (5 + i) % page for i in range(first)]
    used = set(slots)
    rest = [s for s in torch.randperm(pages * page, generator=g).tolist() if s not in used][: n - first]
    slots = torch.tensor(slots + rest, dtype=torch.int32)
    inv = rotary_inv_freq(d, 10000.0, None, d)
    kc = torch.zeros(pages, kv, page, d, dtype=dtype)
    vc = torch.zeros(pages, kv, d, page, dtype=dtype)
    kr, vr = kc.clone(), vc.clone()
    qr = emu.rope_kv_write(qkv, pos, slots, inv, d, 1.0, heads, kv, d, kr, vr, torch.float64)
    kd, vd = kc.to(DEV), vc.to(DEV)
    q = ops.rope_kv_write(qkv.to(DEV), pos.to(DEV), slots.to(DEV), inv.to(DEV), d, 1.0, heads, kv, d, kd, vd, dtype)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    _close(q, qr, tol, "q")
    _close(kd, kr, tol, "k cache")
    _close(vd, vr, tol, "v cache")
    # token by token (the short-step kernel) gives the same bits
    k1, v1 = kc.to(DEV), vc.to(DEV)
    for i in range(0, n, 40):
        ops.rope_kv_write(qkv[i: i + 40].to(DEV), pos[i: i + 40].to(DEV), slots[i: i + 40].to(DEV), inv.to(DEV), d, 1.0,
                          heads, kv, d, k1, v1, dtype)
    assert torch.equal(k1, kd) and torch.equal(v1, vd)


def _attention_case(dtype, heads, kv, d, page, q_lens, ctx_lens, window, seed, allow_fast=True, tune=0, poison=False):
    ops = _ops()
    g = torch.Generator().manual_seed(seed)
    R = len(q_lens)
    n = sum(q_lens)
    pages_needed = sum((c + page - 1) // page for c in ctx_lens)
    pages = pages_needed + 3
    perm = torch.randperm(pages, generator=g).tolist()            # shuffled, non-monotonic tables
    width = max((c + page - 1) // page for c in ctx_lens) + 1
    bt = torch.full((R, width), perm[-1], dtype=torch.int32)
    it = iter(perm)
    for r, c in enumerate(ctx_lens):
        for i in range((c + page - 1) // page):
            bt[r, i] = next(it)
    kc = (torch.randn(pages, kv, page, d, generator=g) * 1.5).to(dtype)
    vc = torch.randn(pages, kv, d, page, generator=g).to(dtype)
    q = (torch.randn(n, heads, d, generator=g) * 1.5).to(dtype)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    cl = torch.tensor(ctx_lens, dtype=torch.int32)
    tr = torch.repeat_interleave(torch.arange(R, dtype=torch.int32), torch.tensor(q_lens))
    scale = 1.0 / math.sqrt(d)
    ref = emu.paged_attention(q, kc, vc, bt, cu, cl, tr, scale, window, max(q_lens), max(ctx_lens)).double()
    if poison:
        # every cache place that holds no key of its request is NaN: the rest of each last page, the spare pages
        used = torch.zeros(pages, page, dtype=torch.bool)
        for r, c in enumerate(ctx_lens):
            for i in range(c):
                used[bt[r, i // page], i % page] = True
        kc = kc.clone()
        vc = vc.clone()
        kc[~used[:, None, :].expand(pages, kv, page)] = float("nan")
        vc.transpose(2, 3)[~used[:, None, :].expand(pages, kv, page)] = float("nan")
    ops.allow_fast_attention = allow_fast
    ops.library().tp_attention_tune(tune)
    try:
        got = ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), cu.to(DEV), cl.to(DEV), tr.to(DEV),
                                  scale, window, max(q_lens), max(ctx_lens))
    finally:
        ops.allow_fast_attention = True
        ops.library().tp_attention_tune(0)
    _close(got, ref, 2e-5 if dtype == torch.float32 else 1.2e-2, f"attention h{heads} kv{kv} d{d} page{page}")
    return got


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,d,page", [(4, 4, 8, 4), (8, 2, 16, 16), (4, 4, 32, 8), (8, 1, 12, 8), (6, 3, 48, 32), (5, 5, 80, 16), (32, 8, 128, 16), (3, 1, 256, 64)])
def test_attention_general(dtype, heads, kv, d, page):
    # ragged: a whole prompt, a portion after a cached prefix, single decoded tokens, a one-token request
    _attention_case(dtype, heads, kv, d, page, [37, 9, 1, 1, 1], [37, 64, 33, 130, 1], 0, seed=5, allow_fast=False)
    _attention_case(dtype, heads, kv, d, page, [20, 1, 6], [50, 77, 6], 13, seed=6, allow_fast=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_far_key_stands_out(dtype):
    """One far key among hundreds carries the whole answer: scale one query/key pair so its score dominates."""
    ops = _ops()
    g = torch.Generator().manual_seed(7)
    heads, kv, d, page, ctx = 4, 2, 64, 16, 700
    pages = (ctx + page - 1) // page
    kc = torch.randn(pages, kv, page, d, generator=g) * 0.1
    vc = torch.randn(pages, kv, d, page, generator=g)
    q = torch.randn(1, heads, d, generator=g) * 0.1
    far = 3                                                 # a key in the first page
    kc[far // page, :, far % page] = q[0, ::2] * 400.0      # aligned with the query of each group's first head
    bt = torch.arange(pages, dtype=torch.int32)[None]
    cu = torch.tensor([0, 1], dtype=torch.int32)
    cl = torch.tensor([ctx], dtype=torch.int32)
    tr = torch.zeros(1, dtype=torch.int32)
    kc, vc, q = kc.to(dtype), vc.to(dtype), q.to(dtype)
    ref = emu.paged_attention(q, kc, vc, bt, cu, cl, tr, 1.0, 0, 1, ctx).double()
    got = ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), cu.to(DEV), cl.to(DEV), tr.to(DEV), 1.0, 0, 1, ctx)
    _close(got, ref, 2e-5 if dtype == torch.float32 else 1.2e-2, "far key")
    # the answer of heads 0 and 2 is (almost) the far key's value row
    assert float((ref.reshape(heads, d)[0] - vc[far // page, 0, :, far % page].double()).abs().max()) < 0.05


@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("m,inter", [(1, 192), (7, 320), (3, 137), (64, 14336)])
def test_swiglu(in_dtype, out_dtype, m, inter):
    ops = _ops()
    g = torch.Generator().manual_seed(8)
    gu = (torch.randn(m, 2 * inter, generator=g) * 4).to(in_dtype)
    gu[0, :4] = torch.tensor([0.0, 80.0, -80.0, 1e4]).to(in_dtype)
    got = ops.swiglu(gu.to(DEV), out_dtype)
    assert torch.isfinite(got.float()).all()
    _close(got, emu.swiglu(gu, torch.float64), _tol(out_dtype), "swiglu")


@pytest.mark.parametrize("m,vocab", [(1, 256), (5, 301), (3, 128256)])
def test_argmax_last_max_wins(m, vocab):
    ops = _ops()
    g = torch.Generator().manual_seed(9)
    lg = torch.randn(m, vocab, generator=g)
    lg[0, 7] = lg[0, vocab - 3] = 50.0                      # an exact tie: the later index wins
    got = ops.argmax(lg.to(DEV)).cpu()
    assert torch.equal(got, emu.argmax(lg))
    assert int(got[0]) == vocab - 3


@pytest.mark.parametrize("m,n,k", [(1, 16, 32), (1, 4096, 4096), (8, 200, 96), (16, 6144, 4096), (17, 48, 64),
                                   (33, 1000, 320), (48, 130, 2048), (64, 4096, 1024), (65, 128, 64),
                                   (200, 300, 96), (257, 384, 160), (512, 1024, 4096),
                                   (300, 333, 192), (513, 130, 64), (700, 1024, 448), (1030, 264, 128), (2048, 128, 320),
                                   (129, 256, 2048), (200, 4096, 4096), (260, 136, 3072), (100, 16400, 128)])
def test_linear_mfma(m, n, k):
    """The matrix-core kernels (decode and prefill shapes) against float64, and against the general kernel."""
    ops = _ops()
    g = torch.Generator().manual_seed(10)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16)
    ref = x.double() @ w.double().T
    xd, wd = x.to(DEV), w.to(DEV)
    got = ops.linear(xd, wd, torch.float32)
    _close(got, ref, 2e-5, "mfma f32 out")
    _close(ops.linear(xd, wd, torch.bfloat16), ref, 1e-2, "mfma bf16 out")
    res = torch.randn(m, n, generator=g)
    _close(ops.linear(xd, wd, torch.float32, residual=res.clone().to(DEV)), ref + res.double(), 2e-5, "mfma residual")
    ops.allow_mfma = False
    try:
        general = ops.linear(xd, wd, torch.float32)
    finally:
        ops.allow_mfma = True
    _close(got, general.double().cpu(), 2e-5, "mfma vs general kernel")
    # a row's result does not depend on the other rows of the batch, beyond the rounding of a
    # different summation order (one row and several rows may take different kernels)
    if m > 1 and m <= 16:
        one = ops.linear(xd[:1].contiguous(), wd, torch.float32)
        _close(one[0], got[0].double().cpu(), 2e-6, "row alone vs in a batch")
        again = ops.linear(xd, wd, torch.float32)
        assert torch.equal(again, got), "the same call must give the same bits"


@pytest.mark.parametrize("m,n,k", [(1, 16, 64), (1, 4096, 4096), (8, 208, 192), (8, 6144, 4096), (16, 1024, 14336), (16, 48, 128),
                                   (17, 48, 64), (33, 1008, 320), (64, 4096, 1024), (100, 16400, 128), (128, 512, 2048),
                                   (129, 256, 2048), (200, 304, 192), (300, 4096, 4096), (700, 1040, 448), (1000, 816, 192),
                                   (2048, 8448, 128), (2100, 6144, 128), (2300, 1024, 256)])
def test_tiled_weights_give_the_same_bits(m, n, k):
    """A weight stored tiled (16 x 32 blocks in the matrix cores' operand order) is the same weight: every product
    that takes it returns the bits it returns for the row-major tensor: plain, bfloat16 out, into a residual, gated,
    with the split norm and k-blocked rows (at most 16 rows), with the partial sums left to the consumer (17..128
    rows) and under both tile sizes of the long products."""
    ops = _ops()
    lib = ops.library()
    g = torch.Generator().manual_seed(21)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
    res = torch.randn(m, n, generator=g).to(DEV)
    t = ops.tile_weight(w)
    assert isinstance(t, ops.TiledWeight) and t.shape == (n, k) and torch.equal(t.row_major(), w)
    assert torch.equal(t.rows(16, n).row_major(), w[16:]) if n > 16 else True
    nw = (torch.rand(n, generator=g) + 0.5).to(DEV)
    for mode in (0, 5, 6) if m > 128 else (0,):
        lib.tp_linear_tune_tile(mode)
        try:
            assert torch.equal(ops.linear(x, t, torch.float32), ops.linear(x, w, torch.float32)), f"f32 out, tile mode {mode}"
            assert torch.equal(ops.linear(x, t, torch.bfloat16), ops.linear(x, w, torch.bfloat16)), f"bf16 out, tile mode {mode}"
            assert torch.equal(ops.linear(x, t, torch.float32, residual=res.clone()),
                               ops.linear(x, w, torch.float32, residual=res.clone())), f"residual, tile mode {mode}"
            a, b = ops.linear_swiglu(x, t, blocked_out=True), ops.linear_swiglu(x, w, blocked_out=True)
            if m <= 16 and (n // 2) % 32 == 0:
                assert isinstance(a, ops.KBlocked) and torch.equal(a.data, b.data), "gated, k-blocked"
            else:
                assert torch.equal(a, b), f"gated, tile mode {mode}"
        finally:
            lib.tp_linear_tune_tile(0)
    if n > 16:      # a slice of whole row groups is a weight of its own
        assert torch.equal(ops.linear(x, ops.weight_rows(t, 16, n), torch.float32), ops.linear(x, w[16:].contiguous(), torch.float32))
    if m <= 128:    # the next norm prepared (at most 16 rows) or the partial sums left to the norm kernel (17..128)
        ra, rb = res.clone(), res.clone()
        ha = ops.linear(x, t, torch.float32, residual=ra, next_norm=(nw, 1e-5))
        hb = ops.linear(x, w, torch.float32, residual=rb, next_norm=(nw, 1e-5))
        assert torch.equal(ra, rb)
        if isinstance(hb[1], ops.Prenormed):
            assert torch.equal(ha[1].x, hb[1].x) and torch.equal(ha[1].ss, hb[1].ss)
            # ... and such rows as the input of the next product
            w2 = torch.randn(64, n, generator=g).to(torch.bfloat16).to(DEV)
            if n % 64 == 0:
                assert torch.equal(ops.linear(ha[1], ops.tile_weight(w2), torch.float32), ops.linear(hb[1], w2, torch.float32))
        elif hb[1] is not None:
            assert torch.equal(ha[1], hb[1])
        pa, pb = ops.linear(x, t, torch.float32, partial_ok=True), ops.linear(x, w, torch.float32, partial_ok=True)
        assert type(pa) is type(pb)
        assert torch.equal(pa.data, pb.data) if isinstance(pa, ops.Partials) else torch.equal(pa, pb)
    if m <= 16 and k % 32 == 0:     # k-blocked rows in
        kb = ops.KBlocked(x.view(m, k // 8, 8).permute(1, 0, 2).contiguous(), m, k)
        assert torch.equal(ops.linear(kb, t, torch.float32), ops.linear(kb, w, torch.float32))


@pytest.mark.parametrize("m,n,k", [(17, 48, 64), (33, 1008, 320), (64, 3072, 3072), (100, 16400, 128), (128, 528, 2048), (60, 4096, 4096)])
def test_linear_mid_rows_both_block_widths(m, n, k):
    """The pipelined product for 17..128 rows with blocks of 128 and of 64 columns, each forced: every output mode
    against float64 (columns that fill no whole block, K split over blocks or not), the partial sums left to the
    next kernel, tiled weights; and the two widths give the same bits (each element's sum runs over K in the
    same order)."""
    ops = _ops()
    lib = ops.library()
    g = torch.Generator().manual_seed(14)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16)
    ref = x.double() @ w.double().T
    res = torch.randn(m, n, generator=g)
    nw = (1 + 0.3 * torch.randn(n, generator=g)).float()
    xd, wd = x.to(DEV), w.to(DEV)
    gate_up = ref.view(m, n // 16, 2, 8)
    gated = (torch.nn.functional.silu(gate_up[:, :, 0]) * gate_up[:, :, 1]).reshape(m, n // 2)
    got = {}
    for width in (2, 1):        # 128 columns, 64 columns
        lib.tp_linear_tune_narrow(width)
        try:
            outs = []
            for wv in (wd, ops.tile_weight(wd)):
                outs.append(ops.linear(xd, wv, torch.float32))
                _close(outs[-1], ref, 2e-5, f"f32 out, width code {width}")
                outs.append(ops.linear(xd, wv, torch.bfloat16))
                _close(outs[-1], ref, 1e-2, f"bf16 out, width code {width}")
                outs.append(ops.linear(xd, wv, torch.float32, residual=res.clone().to(DEV)))
                _close(outs[-1], ref + res.double(), 2e-5, f"residual, width code {width}")
                outs.append(ops.linear_swiglu(xd, wv))
                _close(outs[-1], gated, 1e-2, f"gated, width code {width}")
                h = res.clone().to(DEV)
                handed = ops.linear(xd, wv, torch.float32, residual=h, next_norm=(nw.to(DEV), 1e-5))
                _close(h, ref + res.double(), 2e-5, f"residual with the next norm, width code {width}")
                outs.append(h)
                p = ops.linear(xd, wv, torch.float32, partial_ok=True)
                p = p.data.sum(0)[:m] if isinstance(p, ops.Partials) else p
                _close(p, ref, 2e-5, f"partial sums, width code {width}")
            got[width] = outs
        finally:
            lib.tp_linear_tune_narrow(0)
    for a, b in zip(got[1], got[2]):
        assert torch.equal(a, b), "blocks of 64 and of 128 columns give the same bits"


@pytest.mark.parametrize("m,n,k", [(129, 128, 64), (300, 528, 128), (512, 3072, 3072), (700, 1040, 448), (1000, 816, 192),
                                   (260, 4096, 4096)])
def test_linear_blocks_of_128(m, n, k):
    """The pipelined product on 128 x 128 blocks (what steps of a few hundred rows take when 256 x 128 blocks would
    be too few), forced: every output mode against float64, rows and columns that fill no whole block, K split
    over blocks or not, tiled weights; the bits of the 256 x 128 blocks wherever neither splits K."""
    ops = _ops()
    lib = ops.library()
    g = torch.Generator().manual_seed(15)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16)
    ref = x.double() @ w.double().T
    res = torch.randn(m, n, generator=g)
    xd, wd = x.to(DEV), w.to(DEV)
    gate_up = ref.view(m, n // 16, 2, 8)
    gated = (torch.nn.functional.silu(gate_up[:, :, 0]) * gate_up[:, :, 1]).reshape(m, n // 2)
    got = {}
    for code in (1, 2):          # 128 x 128 always, never
        lib.tp_linear_tune_mid_tile(code)
        try:
            outs = []
            for wv in (wd, ops.tile_weight(wd)):
                outs.append(ops.linear(xd, wv, torch.float32))
                _close(outs[-1], ref, 2e-5, f"f32 out, code {code}")
                outs.append(ops.linear(xd, wv, torch.bfloat16))
                _close(outs[-1], ref, 1e-2, f"bf16 out, code {code}")
                outs.append(ops.linear(xd, wv, torch.float32, residual=res.clone().to(DEV)))
                _close(outs[-1], ref + res.double(), 2e-5, f"residual, code {code}")
                outs.append(ops.linear_swiglu(xd, wv))
                _close(outs[-1], gated, 1e-2, f"gated, code {code}")
            got[code] = outs
        finally:
            lib.tp_linear_tune_mid_tile(0)
    if k // 64 < 32:             # (neither kernel splits a K of fewer than 32 steps)
        for a, b in zip(got[1], got[2]):
            assert torch.equal(a, b), "blocks of 128 x 128 and of 256 x 128 give the same bits"


@pytest.mark.parametrize("m,n,k", [(300, 512, 128), (1000, 816, 192), (257, 256, 64), (2048, 8448, 128), (2100, 6144, 128),
                                   (600, 1152, 320)])
def test_linear_big_tiles(m, n, k):
    """The 256 x 256 block tiles, forced for every whole block of 256 columns (the columns that are left take
    the 256 x 128 tiles in a second launch), and the 256 x 192 tiles, forced wherever N is a multiple of 192:
    every output mode against float64, with rows and columns that fill no whole tile; and the choice the library
    makes by itself at a size where it mixes tiles.  (The size with many tiles and a K loop of two steps is the
    one at which accumulators read too soon after the last MFMA showed as wrong tiles.)"""
    ops = _ops()
    lib = ops.library()
    g = torch.Generator().manual_seed(12)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16)
    ref = x.double() @ w.double().T
    res = torch.randn(m, n, generator=g)
    xd, wd = x.to(DEV), w.to(DEV)
    gate_up = ref.view(m, n // 16, 2, 8)
    gated = (torch.nn.functional.silu(gate_up[:, :, 0]) * gate_up[:, :, 1]).reshape(m, n // 2)
    for mode in (5, 7, 0):
        lib.tp_linear_tune_tile(mode)
        try:
            _close(ops.linear(xd, wd, torch.float32), ref, 2e-5, f"f32 out, tile mode {mode}")
            _close(ops.linear(xd, wd, torch.bfloat16), ref, 1e-2, f"bf16 out, tile mode {mode}")
            _close(ops.linear(xd, wd, torch.float32, residual=res.clone().to(DEV)), ref + res.double(), 2e-5,
                   f"residual, tile mode {mode}")
            _close(ops.linear_swiglu(xd, wd), gated, 1e-2, f"gated, tile mode {mode}")
        finally:
            lib.tp_linear_tune_tile(0)


@pytest.mark.parametrize("m,hidden,kp,nc", [(1, 64, 32, 48), (8, 4096, 4096, 6144), (16, 160, 96, 272), (5, 4096, 14336, 1024),
                                             (3, 96, 2048, 40)])
def test_linear_split_norm(m, hidden, kp, nc):
    """A norm carried by the products around it: the product that adds into the residual stream prepares
    (rows times norm weight in bfloat16, sums of squares per 16 columns), the next product applies the
    scale to its float32 sums.  Against float64, and against the norm kernel followed by the plain product."""
    ops = _ops()
    g = torch.Generator().manual_seed(30)
    eps = 1e-5
    h = torch.randn(m, hidden, generator=g) * 3
    a = torch.randn(m, kp, generator=g).to(torch.bfloat16)
    wo = (torch.randn(hidden, kp, generator=g) * 0.05).to(torch.bfloat16)
    nw = (1 + 0.3 * torch.randn(hidden, generator=g)).float()
    wc = (torch.randn(nc, hidden, generator=g) * 0.1).to(torch.bfloat16)
    assert ops.split_norm_ok(m, hidden, torch.bfloat16)
    h2_ref = h.double() + a.double() @ wo.double().T
    hd = h.clone().to(DEV)
    out, pre = ops.linear(a.to(DEV), wo.to(DEV), torch.float32, residual=hd, next_norm=(nw.to(DEV), eps))
    assert out is hd and pre is not None
    _close(hd, h2_ref, 2e-5, "residual")
    assert torch.equal(pre.rows().cpu(), (hd.cpu() * nw).to(torch.bfloat16)), "rows times norm weight, rounded once"
    ss = pre.ss.cpu().double().sum(0)[:m]
    assert float(((ss - (hd.cpu().double() ** 2).sum(1)).abs() / ss).max()) < 1e-5
    normed = h2_ref * torch.rsqrt((h2_ref ** 2).mean(1, keepdim=True) + eps) * nw.double()
    ref = normed @ wc.double().T
    got = ops.linear(pre, wc.to(DEV), torch.float32)
    _close(got, ref, 6e-3, "consumer of the handed-over rows")
    plain = ops.linear(ops.rmsnorm(hd, nw.to(DEV), eps, torch.bfloat16), wc.to(DEV), torch.float32)
    _close(got, plain.double().cpu(), 6e-3, "split norm vs norm kernel + product")
    if nc % 16 == 0:
        gu = ref.reshape(m, -1, 2, 8)
        gt, up = gu[:, :, 0].reshape(m, -1), gu[:, :, 1].reshape(m, -1)
        _close(ops.linear_swiglu(pre, wc.to(DEV)), gt / (1 + torch.exp(-gt)) * up, 1e-2, "gated consumer")
    # sizes that do not allow it: the product still adds, and says that the norm has to run on its own
    if hidden % 32 == 0:
        a2 = torch.randn(m, 24, generator=g).to(torch.bfloat16)
        w2 = torch.randn(hidden, 24, generator=g).to(torch.bfloat16)
        h3 = hd.clone()
        out, none = ops.linear(a2.to(DEV), w2.to(DEV), torch.float32, residual=h3, next_norm=(nw.to(DEV), eps))
        assert none is None
        _close(h3, hd.double().cpu() + a2.double() @ w2.double().T, 2e-5, "fallback product")


@pytest.mark.parametrize("m,hidden,kp", [(17, 256, 1024), (64, 4096, 4096), (100, 160, 2048), (128, 512, 256),
                                         (300, 1024, 2048), (512, 4096, 4096), (700, 3072, 8192), (1000, 512, 4096)])
def test_linear_deferred_reduction(m, hidden, kp):
    """Products with few result tiles split K over blocks; the partial sums may stay unadded for the next kernel:
    the one that adds them into the residual stream and norms it, or the rotation and cache write."""
    ops = _ops()
    g = torch.Generator().manual_seed(31)
    eps = 1e-5
    h = torch.randn(m, hidden, generator=g) * 3
    a = torch.randn(m, kp, generator=g).to(torch.bfloat16)
    wo = (torch.randn(hidden, kp, generator=g) * 0.05).to(torch.bfloat16)
    nw = (1 + 0.3 * torch.randn(hidden, generator=g)).float()
    assert ops.split_norm_ok(m, hidden, torch.bfloat16)
    # residual product + norm in one go, against the three kernels it replaces
    h_plain = ops.linear(a.to(DEV), wo.to(DEV), torch.float32, residual=h.clone().to(DEV))
    x_plain = ops.rmsnorm(h_plain, nw.to(DEV), eps, torch.bfloat16)
    hd = h.clone().to(DEV)
    out, x = ops.linear(a.to(DEV), wo.to(DEV), torch.float32, residual=hd, next_norm=(nw.to(DEV), eps))
    assert out is hd
    _close(hd, h.double() + a.double() @ wo.double().T, 2e-5, "residual")
    if x is None:                      # K too short to be split: the product wrote the residual itself
        assert torch.equal(hd, h_plain)
    else:
        assert torch.equal(hd, h_plain), "the same sums in the same order"
        h64 = hd.double().cpu()
        want = h64 * torch.rsqrt((h64 ** 2).mean(1, keepdim=True) + eps) * nw.double()
        assert x.dtype == torch.bfloat16
        _close(x, want, 5e-3, "normed rows")            # (the sum of squares runs in another order than the norm kernel's)
        _close(x, x_plain.double().cpu(), 1e-2, "fused against the norm kernel")
    # projection whose partial sums the rotation adds
    heads, kvh, d, ps = 4, 2, 32, 16
    width = (heads + 2 * kvh) * d
    xin = torch.randn(m, hidden, generator=g).to(torch.bfloat16)
    wqkv = (torch.randn(width, hidden, generator=g) * 0.05).to(torch.bfloat16)
    pos = torch.arange(3, 3 + m, dtype=torch.int32)
    slots = torch.randperm(m * 2, generator=g)[:m].to(torch.int32)
    inv_freq = (1.0 / 10000.0 ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    pages = (m * 2 + ps - 1) // ps
    results = []
    for partial_ok in (False, True):
        kc = torch.zeros(pages, kvh, ps, d, dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros(pages, kvh, d, ps, dtype=torch.bfloat16, device=DEV)
        qkv = ops.linear(xin.to(DEV), wqkv.to(DEV), torch.float32, partial_ok=partial_ok)
        if partial_ok and hidden >= 1024 and (m <= 128 or hidden >= 2048):
            assert isinstance(qkv, ops.Partials) and qkv.shape == (m, width)
        q = ops.rope_kv_write(qkv, pos.to(DEV), slots.to(DEV), inv_freq.to(DEV), d, 1.0, heads, kvh, d, kc, vc, torch.bfloat16)
        results.append((q, kc, vc))
    for u, v in zip(results[0], results[1]):
        assert torch.equal(u, v), "adding the partial sums in the next kernel changes nothing"


@pytest.mark.parametrize("heads,kv,d,page", [(4, 2, 32, 8), (8, 2, 64, 16), (6, 3, 96, 32), (32, 8, 128, 16), (8, 8, 128, 64),
                                             (20, 1, 64, 16), (5, 1, 128, 8)])
def test_attention_mfma(heads, kv, d, page):
    """The matrix-core kernels: portions (with and without a cached prefix) beside single decoded tokens."""
    bf = torch.bfloat16
    _attention_case(bf, heads, kv, d, page, [37, 9, 1, 1, 1], [37, 64, 33, 130, 1], 0, seed=11)      # mixed
    _attention_case(bf, heads, kv, d, page, [1, 1, 1], [700, 31, 257], 0, seed=12)                     # decode only, split context
    _attention_case(bf, heads, kv, d, page, [70, 33], [70, 97], 0, seed=13)                            # portions only
    _attention_case(bf, heads, kv, d, page, [20, 1, 6, 1], [50, 77, 6, 300], 13, seed=14)              # window
    _attention_case(bf, heads, kv, d, page, [40, 1], [200, 200], 64, seed=15)                          # window longer than a step
    # a wave takes 32 query rows when there are many blocks and 16 when there are few: the same bits
    for q_lens, ctx_lens, window in (([70, 33, 1], [70, 97, 40], 0), ([45, 100], [300, 100], 50)):
        a, b = (_attention_case(bf, heads, kv, d, page, q_lens, ctx_lens, window, seed=17, tune=t) for t in (2, 3))
        assert torch.equal(a, b)


@pytest.mark.parametrize("heads,kv,d,page", [(8, 2, 128, 16), (6, 3, 64, 32), (5, 1, 32, 64)])
def test_attention_portions_with_split_keys(heads, kv, d, page):
    """Few query blocks under a long context: the keys of a portion are split over blocks and the parts combined.
    Parts of at least 64 keys here, so that there are many (query blocks with few steps get fewer parts, or stay
    whole and write their rows themselves), beside single decoded tokens, with and without a window; the unsplit
    kernel's result is within rounding."""
    ops = _ops()
    bf = torch.bfloat16
    cases = (([40, 1, 5, 1], [700, 300, 41, 64], 0), ([33, 2], [1000, 515], 0), ([70, 1], [900, 130], 300))
    keep = ops.portion_min_keys, ops.portion_target_blocks
    try:
        for q_lens, ctx_lens, window in cases:
            ops.portion_min_keys, ops.portion_target_blocks = 64, 4096
            a = _attention_case(bf, heads, kv, d, page, q_lens, ctx_lens, window, seed=18)
            ops.portion_target_blocks = 1
            b = _attention_case(bf, heads, kv, d, page, q_lens, ctx_lens, window, seed=18)
            assert not torch.equal(a, b), "the split path did not run"
            _close(a, b.double().cpu(), 8e-3, "split against unsplit")
    finally:
        ops.portion_min_keys, ops.portion_target_blocks = keep


@pytest.mark.parametrize("dtype,fast,heads,kv,d,page", [(torch.bfloat16, True, 8, 2, 128, 16), (torch.bfloat16, True, 6, 3, 96, 32),
                                                        (torch.bfloat16, True, 4, 2, 64, 8), (torch.bfloat16, True, 5, 1, 32, 64),
                                                        (torch.bfloat16, False, 4, 2, 48, 16), (torch.float32, False, 4, 2, 80, 16)])
def test_attention_ignores_what_lies_past_the_last_key(dtype, fast, heads, kv, d, page):
    """A page keeps what its previous owner wrote; if that was not finite, nothing of it may reach the new
    owner: NaN in every cache place that holds no key (the matrix-core kernels fetch eight key places of a value
    at once, and 0 * NaN is NaN)."""
    for q_lens, ctx_lens, window in (([37, 9, 1, 1, 1], [37, 61, 33, 130, 1], 0), ([1, 1, 1], [700, 31, 257], 0),
                                     ([70, 33], [70, 97], 0), ([20, 1, 6, 1], [50, 77, 6, 300], 13)):
        got = _attention_case(dtype, heads, kv, d, page, q_lens, ctx_lens, window, seed=21, allow_fast=fast, poison=True)
        assert bool(torch.isfinite(got.float()).all())


@pytest.mark.parametrize("heads,kv,d,page", [(5, 1, 32, 8), (6, 2, 96, 16), (4, 2, 64, 16), (8, 2, 128, 16)])
def test_attention_decode_with_more_than_32_splits(heads, kv, d, page):
    """One request of 5,000 keys is cut into 39 splits (one for every 128 keys) where few blocks would otherwise run:
    the kernel that adds the splits hands each split's weight from lane to lane, which every lane has to take part
    in also for head sizes below 64 (a lane that sat out once left the later splits' weights undefined)."""
    ops = _ops()
    keep = ops.decode_target_blocks
    try:
        ops.decode_target_blocks = 4096
        _attention_case(torch.bfloat16, heads, kv, d, page, [1], [5000], 0, seed=24)
        _attention_case(torch.bfloat16, heads, kv, d, page, [1, 1], [4999, 2300], 700, seed=25)
    finally:
        ops.decode_target_blocks = keep


def test_attention_mfma_long_decode():
    _attention_case(torch.bfloat16, 8, 2, 128, 16, [1, 1], [3000, 2049], 0, seed=16)


@pytest.mark.parametrize("dtype,fast", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
def test_attention_window_edge(dtype, fast):
    """Two keys carry huge scores: the one exactly at the window's edge (position p - w + 1) must be seen,
    the one just outside (p - w) must not.  A window off by one in either direction changes the answer."""
    ops = _ops()
    g = torch.Generator().manual_seed(17)
    heads, kv, d, page, ctx, w = 2, 1, 64, 16, 200, 37
    pages = (ctx + page - 1) // page
    q = torch.randn(1, heads, d, generator=g) * 0.1
    kc = torch.randn(pages, kv, page, d, generator=g) * 0.1
    vc = torch.randn(pages, kv, d, page, generator=g)
    pos = ctx - 1
    edge, outside = pos - w + 1, pos - w
    for j, gain in ((edge, 300.0), (outside, 600.0)):
        kc[j // page, 0, j % page] = q[0, 0] * gain
    bt = torch.arange(pages, dtype=torch.int32)[None]
    cu = torch.tensor([0, 1], dtype=torch.int32)
    cl = torch.tensor([ctx], dtype=torch.int32)
    tr = torch.zeros(1, dtype=torch.int32)
    q, kc, vc = q.to(dtype), kc.to(dtype), vc.to(dtype)
    ref = emu.paged_attention(q, kc, vc, bt, cu, cl, tr, 1.0, w, 1, ctx).double()
    assert float((ref.reshape(heads, d)[0] - vc[edge // page, 0, :, edge % page].double()).abs().max()) < 0.05
    ops.allow_fast_attention = fast
    try:
        got = ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), cu.to(DEV), cl.to(DEV), tr.to(DEV), 1.0, w, 1, ctx)
    finally:
        ops.allow_fast_attention = True
    _close(got, ref, 2e-5 if dtype == torch.float32 else 1.2e-2, "window edge")


@pytest.mark.parametrize("m,inter,k", [(1, 192, 64), (8, 14336, 4096), (16, 320, 96), (40, 136, 160), (4, 136, 160), (64, 1024, 2048), (300, 200, 128), (2048, 512, 256), (515, 328, 64), (160, 256, 2048)])
def test_linear_swiglu(m, inter, k):
    """The gated epilogue of the matrix-core products, on the interleaved gate/up layout."""
    ops = _ops()
    g = torch.Generator().manual_seed(20)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    wg = (torch.randn(inter, k, generator=g) * 0.3).to(torch.bfloat16)
    wu = (torch.randn(inter, k, generator=g) * 0.3).to(torch.bfloat16)
    w = ops.interleave_gate_up(wg, wu)
    assert torch.equal(w[:8], wg[:8]) and torch.equal(w[8:16], wu[:8]) and torch.equal(w[16:24], wg[8:16])
    gd, ud = x.double() @ wg.double().T, x.double() @ wu.double().T
    ref = gd / (1 + torch.exp(-gd)) * ud
    got = ops.linear_swiglu(x.to(DEV), w.to(DEV))
    assert got.shape == (m, inter)
    _close(got, ref, 6e-3, "linear_swiglu")
    assert torch.equal(emu.linear_swiglu(x, w), ref.to(torch.bfloat16))
    # k-blocked output for a few rows: the same numbers in the other layout, and the product that takes them
    blk = ops.linear_swiglu(x.to(DEV), w.to(DEV), blocked_out=True)
    if m > 16 or inter % 32:
        assert torch.is_tensor(blk) and torch.equal(blk, got)     # (the product that takes k-blocked rows steps K by 32)
    else:
        assert tuple(blk.data.shape) == (inter // 8, m, 8) and blk.shape == (m, inter)
        assert torch.equal(blk.row_major(), got)
        assert torch.equal(emu.linear_swiglu(x, w, True).data, ref.to(torch.bfloat16).reshape(m, inter // 8, 8).permute(1, 0, 2))
        w2 = (torch.randn(72, inter, generator=g) * 0.2).to(torch.bfloat16)
        res = torch.randn(m, 72, generator=g)
        want = res.double() + got.double().cpu() @ w2.double().T
        r1 = res.clone().to(DEV)
        ops.linear(blk, w2.to(DEV), torch.float32, residual=r1)
        _close(r1, want, 2e-5, "product of k-blocked rows")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seed,n,mean,std", [(0, 1, 0.0, 0.02), (7, 4_000_037, 0.0, 0.02), (2 ** 63 + 11, 1_000_000, 1.0, 0.2)])
def test_fill_normal_has_the_host_generator_s_bits(dtype, seed, n, mean, std):
    """The device kernel, the host library and the numpy twin (tests/plain_random.py) agree on every element."""
    import numpy as np
    import plain_random
    from tempura_amd.weights.random_init import fill_normal_host
    ops = _ops()
    dev = ops.fill_normal(torch.empty(n, dtype=dtype, device=DEV), seed, mean, std).cpu()
    host = fill_normal_host(torch.empty(n, dtype=dtype), seed, mean, std)
    assert torch.equal(dev.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       host.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    twin = torch.from_numpy(plain_random.fill_normal((min(n, 300_000),), seed, mean, std)).to(dtype)
    assert torch.equal(dev[: twin.numel()], twin)


def test_device_made_model_equals_the_written_folder(tmp_path):
    """A model made in device memory holds the weights of the folder written from the same configuration and seed."""
    import helpers
    from tempura_amd.config import LlamaConfig
    from tempura_amd.engine.loading import load_model, random_model
    _ops()
    cfg = LlamaConfig.from_dict(helpers.CONFIGS["D"].to_dict())
    from tempura_amd.weights import write_random_model
    for dtype in ("float32", "bfloat16"):
        d = write_random_model(cfg, str(tmp_path / dtype), seed=5, std=0.1, norm_jitter=0.1, dtype=dtype)
        a = load_model(d, dtype, DEV)
        b = random_model(cfg, seed=5, dtype=dtype, device=DEV, std=0.1, norm_jitter=0.1)
        for la, lb in zip(a.layers, b.layers):
            for pa, pb in zip(la.parts(), lb.parts()):
                for key, va in vars(pa).items():
                    vb = getattr(pb, key)
                    va, vb = getattr(va, "data", va), getattr(vb, "data", vb)
                    if isinstance(va, torch.Tensor):
                        assert torch.equal(va, vb), f"{type(pa).__name__}.{key} differs ({dtype})"
        assert torch.equal(a.embedding.weight, b.embedding.weight) and torch.equal(a.final_norm.weight, b.final_norm.weight)


@pytest.mark.parametrize("dtype", [torch.float32, torch.int32])
@pytest.mark.parametrize("n,width", [(1, 1), (7, 301), (64, 128256), (5, 1024), (3, 1025)])
def test_take_rows_and_zero_rows(dtype, n, width):
    ops = _ops()
    g = torch.Generator().manual_seed(n + width)
    src = (torch.randn(n, width, generator=g) * 100).to(dtype)
    d = src.to(DEV)
    rows = [int(r) for r in torch.randint(0, n, (max(1, n // 2 + 1),), generator=g)]
    assert torch.equal(ops.take_rows(d, rows).cpu(), src[rows])
    assert torch.equal(ops.take_rows(d).cpu(), src) and ops.take_rows(d).data_ptr() != d.data_ptr()
    assert torch.equal(ops.take_rows(d[:, 0].contiguous(), rows).cpu(), src[rows, 0])
    assert ops.take_rows(d, []).shape == (0, width)
    ops.zero_rows(d, sorted(set(rows)))
    want = src.clone()
    want[sorted(set(rows))] = 0
    assert torch.equal(d.cpu(), want)
    with pytest.raises(Exception, match="out of range"):
        ops.take_rows(d, [n])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_pages_beyond_two_to_the_31_elements_of_a_pool(dtype):
    """A layer's key (or value) pool may hold more than 2^31 elements (4 GiB of bfloat16: 2.1 million tokens of 8 kv
    heads of 128, which a small model's cache reaches on this GPU): every kernel that writes or reads the cache works
    out its places in 64 bits.  The same step is run twice, on a small pool and on pages that all lie past element
    2^31 of a large one (a block table with the same pages plus an offset): the rows that the rotation and
    cache-write kernels store (few rows and a long step, alone and as a projection's epilogue), and what attention
    then reads for a prompt and for single tokens, must be the same bits."""
    ops = _ops()
    from tempura_amd.parts.rope import rotary_inv_freq
    heads, kv, d, page, hidden = 32, 8, 128, 16, 128
    small = 150
    off = 2 ** 31 // (kv * page * d) + 3                   # the first page of the large pool that is used
    big = off + small
    g = torch.Generator().manual_seed(11)
    n = (heads + 2 * kv) * d
    inv = rotary_inv_freq(d, 500000.0, None, d).to(DEV)
    w = (torch.randn(n, hidden, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    m_long, m_few = 2100, 8
    x_long = torch.randn(m_long, hidden, generator=g).to(torch.bfloat16).to(DEV)
    x_few = torch.randn(m_few, hidden, generator=g).to(torch.bfloat16).to(DEV)
    order = torch.randperm(small - 1, generator=g).tolist()            # (the last page stays the tables' filler)
    sl_long = torch.tensor([order[i // page] * page + i % page for i in range(m_long)], dtype=torch.int32)
    rest = order[(m_long + page - 1) // page:]
    sl_few = torch.tensor([rest[i] * page + (5 * i) % page for i in range(m_few)], dtype=torch.int32)
    pos_long = torch.arange(m_long, dtype=torch.int32).to(DEV)
    pos_few = torch.randint(0, 100000, (m_few,), generator=g, dtype=torch.int32).to(DEV)
    # attention afterwards: the prompt as one request, and four requests of one token over parts of its pages
    width = (m_long + page - 1) // page + 1
    bt_prompt = torch.full((1, width), small - 1, dtype=torch.int32)
    bt_prompt[0, : width - 1] = torch.tensor(order[: width - 1], dtype=torch.int32)
    ctx_single = [m_long, 1500, 333, 17]
    bt_single = bt_prompt.repeat(4, 1)
    q_single = (torch.randn(4, heads, d, generator=g) * 1.5).to(dtype).to(DEV)
    scale = 1.0 / math.sqrt(d)

    def run(pages, shift):
        kc = torch.empty(pages, kv, page, d, dtype=dtype, device=DEV)
        vc = torch.empty(pages, kv, d, page, dtype=dtype, device=DEV)
        kc[shift: shift + small].zero_()
        vc[shift: shift + small].zero_()
        a, b = (sl_long + shift * page).to(DEV), (sl_few + shift * page).to(DEV)
        outs = []
        if dtype == torch.bfloat16:    # the projections whose epilogue rotates and stores
            outs.append(ops.linear_rope_kv(x_long, w, pos_long, a, inv, d, 1.0, heads, kv, d, kc, vc, ops.rope_table(pos_long, inv, d, 1.0)))
            outs.append(ops.linear_rope_kv(x_few, w, pos_few, b, inv, d, 1.0, heads, kv, d, kc, vc))
        else:                          # the kernels of their own, for a long step and for a few rows
            outs.append(ops.rope_kv_write(ops.linear(x_long.float(), w.float(), torch.float32), pos_long, a, inv, d, 1.0, heads, kv, d, kc, vc, dtype))
            outs.append(ops.rope_kv_write(ops.linear(x_few.float(), w.float(), torch.float32), pos_few, b, inv, d, 1.0, heads, kv, d, kc, vc, dtype))
        q_prompt = outs[0].to(dtype).view(m_long, heads, d)
        cu = torch.tensor([0, m_long], dtype=torch.int32, device=DEV)
        outs.append(ops.paged_attention(q_prompt, kc, vc, (bt_prompt + shift).to(DEV), cu, torch.tensor([m_long], dtype=torch.int32, device=DEV),
                                        torch.zeros(m_long, dtype=torch.int32, device=DEV), scale, 0, m_long, m_long))
        outs.append(ops.paged_attention(q_single, kc, vc, (bt_single + shift).to(DEV), torch.arange(5, dtype=torch.int32, device=DEV),
                                        torch.tensor(ctx_single, dtype=torch.int32, device=DEV), torch.arange(4, dtype=torch.int32, device=DEV),
                                        scale, 0, 1, max(ctx_single)))
        outs += [kc[shift: shift + small].clone(), vc[shift: shift + small].clone()]
        return outs

    assert big * kv * page * d > 2 ** 31 and off * kv * page * d >= 2 ** 31
    low = run(small, 0)
    high = run(big, off)
    names = ["q of the long step", "q of the few rows", "attention of the prompt", "attention of single tokens", "key pages", "value pages"]
    for name, x0, x1 in zip(names, low, high):
        assert torch.isfinite(x0.float()).all(), name
        assert torch.equal(x0, x1), f"{name}: other bits on pages past element 2^31"
