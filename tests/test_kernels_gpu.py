"""Each kernel alone against a plain torch reference of the same op, at other sizes than the
engine tests use (among them the 7B model's).  The tuned bf16 kernels are also compared with
their plain kernels."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def ops():
    from flambeau_amd.kernels import ops as o
    return o


def tuned():
    from flambeau_amd.kernels import tuned as t
    return t


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


# ---------------------------------------------------------------- element-wise and norm kernels
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V,H,n", [(300, 80, 7), (32768, 4096, 33), (5, 3, 1)])
def test_embed(dtype, V, H, n):
    table = rnd(V, H, dtype=dtype)
    tokens = torch.randint(0, V, (n,), dtype=torch.int32, device=DEV)
    out = torch.empty(n, H, dtype=torch.float32, device=DEV)
    ops().embed(table, tokens, out)
    assert torch.equal(out, table[tokens.long()].float())


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,H,eps", [(5, 96, 1e-6), (3, 4096, 1e-5), (17, 250, 1e-2), (2, 5120, 1e-5)])
def test_rmsnorm_variants(out_dtype, n, H, eps):
    x = rnd(n, H, seed=1)
    d = rnd(n, H, seed=2, scale=0.3)
    w = 1 + 0.1 * rnd(H, seed=3)
    tol = 1e-5 if out_dtype == torch.float32 else 1e-2

    def ref(v):
        v = v.double()
        return (v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w.double())

    out = torch.empty(n, H, dtype=out_dtype, device=DEV)
    ops().rmsnorm(x, w, out, eps)
    assert (out.double() - ref(x)).abs().max() < tol * ref(x).abs().max()
    # with the pending delta added and stored back
    x2 = x.clone()
    ops().rmsnorm(x2, w, out, eps, delta=d, store_sum=True)
    assert torch.equal(x2, x + d)
    assert (out.double() - ref(x + d)).abs().max() < tol * ref(x + d).abs().max()
    # gathered rows, nothing stored
    rows = torch.tensor([n - 1, 0, n // 2], dtype=torch.int32, device=DEV)
    out3 = torch.empty(3, H, dtype=out_dtype, device=DEV)
    x3 = x.clone()
    ops().rmsnorm(x3, w, out3, eps, delta=d, rows=rows)
    assert torch.equal(x3, x)
    assert (out3.double() - ref(x + d)[rows.long()]).abs().max() < tol * ref(x + d).abs().max()


def test_add_and_silu_mul():
    x, d = rnd(37, 1000, seed=4), rnd(37, 1000, seed=5)
    want = x + d
    ops().add_inplace(x, d)
    assert torch.equal(x, want)
    for n, I in [(3, 224), (9, 14336), (1, 5)]:
        gu = rnd(n, 2 * I, seed=6, scale=3.0)
        ref = (gu[:, :I].double() / (1 + torch.exp(-gu[:, :I].double()))) * gu[:, I:].double()
        o32 = torch.empty(n, I, dtype=torch.float32, device=DEV)
        ops().silu_mul(gu, o32)
        assert torch.allclose(o32.double(), ref, rtol=2e-6, atol=1e-6)     # float32 rounding of values up to 100
        o16 = torch.empty(n, I, dtype=torch.bfloat16, device=DEV)
        ops().silu_mul(gu, o16)
        assert (o16.double() - ref).abs().max() < 1e-2 * ref.abs().max()


# ---------------------------------------------------------------- matrix products
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (7, 100, 36), (65, 130, 250), (33, 384, 96), (2, 6144, 4096)])
def test_gemm_plain_float32(M, N, K):
    x, w = rnd(M, K, seed=7), rnd(N, K, seed=8)
    out = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops().gemm_plain(x, w, out)
    ref = x.double() @ w.double().T
    assert (out.double() - ref).abs().max() < 2e-6 * math.sqrt(K) * ref.abs().max().clamp(min=1)


def test_gemm_plain_rows_do_not_depend_on_the_batch():
    x, w = rnd(70, 300, seed=9), rnd(200, 300, seed=10)
    full = torch.empty(70, 200, dtype=torch.float32, device=DEV)
    ops().gemm_plain(x, w, full)
    one = torch.empty(1, 200, dtype=torch.float32, device=DEV)
    ops().gemm_plain(x[41:42].contiguous(), w, one)
    assert torch.equal(one[0], full[41])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (8, 6144, 4096), (1, 4096, 14336), (64, 1024, 512),
                                   (3, 100, 72), (17, 250, 40), (5, 16, 8), (33, 28672, 4096), (1, 32768, 4096),
                                   (16, 37, 264), (49, 300, 80)])
def test_gemm_skinny_against_plain(out_dtype, M, N, K):
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=11), rnd(N, K, dtype=torch.bfloat16, seed=12, scale=0.05)
    from flambeau_amd.kernels.packing import pack_weight, unpack_weight
    packed = pack_weight(w)
    assert torch.equal(unpack_weight(packed, N, K), w)
    got = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    tuned().gemm_skinny(x, packed, got)
    ref = x.double() @ w.double().T
    plain = torch.empty(M, N, dtype=out_dtype, device=DEV)
    ops().gemm_plain(x, w, plain)
    scale = ref.abs().max()
    tol = 1e-5 if out_dtype == torch.float32 else 5e-3
    assert (got.double() - ref).abs().max() < tol * scale
    assert (got.double() - plain.double()).abs().max() < 2 * tol * scale


@pytest.mark.parametrize("M,N,K", [(1, 80, 96), (7, 48, 1024), (5, 37, 264), (16, 6144, 512), (12, 4112, 72), (9, 16400, 2560), (8, 4096, 14336),
                                   (12, 1024, 4096), (6, 1024, 4096)])
def test_gemm_skinny_with_several_row_groups_per_block(M, N, K):
    """One or two row groups per block (the last block may hold one), x fetched piece by piece or by
    rows through LDS, and any number of waves give the same numbers as long as K is split over the
    same number of waves; plain and SwiGLU epilogue."""
    from flambeau_amd.kernels.packing import pack_weight
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=13), rnd(N, K, dtype=torch.bfloat16, seed=14, scale=0.05)
    packed = pack_weight(w)
    ref = x.double() @ w.double().T
    for waves in (0, 2, 4, 8, 16):                    # 0: the kernel's own choice
        outs = []
        for groups in (1, 2):
            for direct_x in (0, 1):
                got = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
                tuned().gemm_skinny(x, packed, got, waves + 256 * groups + 65536 * direct_x)
                assert (got.double() - ref).abs().max() < 1e-5 * ref.abs().max()
                outs.append(got)
        if waves in (2, 4, 8) and K // 32 >= 2 * waves:       # (fewer steps than that: the kernel takes fewer waves)
            assert all(torch.equal(outs[0], o) for o in outs[1:])
    if N % 32 == 0:
        gate, up = w[:N // 2].contiguous(), w[N // 2:].contiguous()
        Wgu = tuned().prepare_gate_up(gate, up)
        gr, ur = x.double() @ gate.double().T, x.double() @ up.double().T
        ref_act = gr / (1 + torch.exp(-gr)) * ur
        for groups in (1, 2):
            act = torch.full((M, N // 2), float("nan"), dtype=torch.float32, device=DEV)
            tuned().gemm_skinny(x, Wgu.packed, act, 256 * groups, swiglu_rows=Wgu.packed_rows)
            assert (act.double() - ref_act).abs().max() < 1e-5 * ref_act.abs().max()
    with pytest.raises(Exception, match="row groups"):
        tuned().gemm_skinny(x, packed, torch.empty(M, N, dtype=torch.float32, device=DEV), 256 * 3)


@pytest.mark.parametrize("M,H,N2,I,eps", [(1, 4096, 6144, 512, 1e-5), (8, 4096, 32768, 14336, 1e-5), (16, 72, 40, 104, 1e-2),
                                            (8, 5104, 6144, 96, 1e-5), (12, 5120, 28672, 256, 1e-5),
                                            (3, 136, 250, 40, 1e-6), (5, 64, 16, 8, 1e-5),
                                            (64, 4096, 6144, 14336, 1e-5), (17, 96, 40, 64, 1e-3), (40, 2080, 300, 160, 1e-5),
                                            (2048, 4096, 1024, 512, 1e-5), (300, 264, 152, 96, 1e-6), (129, 72, 40, 104, 1e-3),
                                            (128, 4096, 6144, 4096, 1e-5), (100, 520, 64, 2048, 1e-5), (512, 5120, 256, 1024, 1e-5)])
def test_gemm_fused_with_the_norms_around_it(M, H, N2, I, eps):
    from flambeau_amd.kernels import KernelError
    """resid += a W1^T in the product's epilogue, norm(resid) W2^T through the row scale of the next
    product, against the same chain in float64; and the SwiGLU epilogue after a row scale.  Up to 16
    rows in the skinny kernel, 17 to 64 in the kernel that shares x through LDS, more in the tiled one."""
    from flambeau_amd.kernels.packing import pack_weight
    a = rnd(M, I, dtype=torch.bfloat16, seed=51)
    w1 = rnd(H, I, dtype=torch.bfloat16, seed=52, scale=0.05)
    w2 = rnd(N2, H, dtype=torch.bfloat16, seed=53, scale=0.05)
    g = rnd(H, seed=54).abs() + 0.5
    resid0 = rnd(M, H, seed=55)
    resid = resid0.clone()
    xg = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    if M <= 16:
        ssq = torch.full((M, tuned().skinny_parts(H)), float("nan"), dtype=torch.float32, device=DEV)
        rows = tuned().gemm_skinny_residual(a, pack_weight(w1), resid, g, xg, ssq, eps)
    elif M <= 64:
        ssq = torch.full((M, tuned().mid_parts(H)), float("nan"), dtype=torch.float32, device=DEV)
        ws = torch.full((tuned().gemm_mid_splits(M, H, I) * M * H,), float("nan"), dtype=torch.float32, device=DEV)
        rows = tuned().gemm_mid_residual(a, pack_weight(w1), resid, g, xg, ssq, eps, ws)
    else:
        splits = tuned().gemm_tiled_splits(M, H, I)
        ws = torch.full((splits * M * H,), float("nan"), dtype=torch.float32, device=DEV) if splits > 1 else None
        if splits > 1:
            with pytest.raises(KernelError, match="workspace"):
                tuned().gemm_tiled_residual(a, pack_weight(w1), resid, g, xg, torch.empty(M, tuned().tiled_parts(M, H, I), device=DEV), eps)
        ssq = torch.full((M, tuned().tiled_parts(M, H, I)), float("nan"), dtype=torch.float32, device=DEV)
        rows = tuned().gemm_tiled_residual(a, pack_weight(w1), resid, g, xg, ssq, eps, ws)
    r_ref = resid0.double() + a.double() @ w1.double().T
    assert (resid.double() - r_ref).abs().max() < 1e-5 * r_ref.abs().max()
    assert (ssq.double().sum(1) - (r_ref ** 2).sum(1)).abs().max() < 1e-5 * (r_ref ** 2).sum(1).max()
    assert (xg.double() - r_ref * g.double()).abs().max() < 5e-3 * (r_ref * g.double()).abs().max()
    normed = r_ref * torch.rsqrt((r_ref ** 2).mean(1, keepdim=True) + eps) * g.double()
    ref = normed @ w2.double().T
    class Rt:
        def buffer(self, name, n, cols, dtype=torch.bfloat16, max_rows=None):
            return torch.empty(n, cols, dtype=dtype, device=DEV)
    W2 = tuned().prepare_weight(w2)
    got = torch.full((M, N2), float("nan"), dtype=torch.float32, device=DEV)
    tuned().gemm(rows, W2, got, Rt())
    assert (got.double() - ref).abs().max() < 6e-3 * ref.abs().max()
    # the rows themselves, for kernels that do not take the factors
    made = rows.materialize(Rt())
    assert (made.double() - normed).abs().max() < 5e-3 * normed.abs().max()
    if N2 % 32 == 0:
        gate, up = w2[:N2 // 2].contiguous(), w2[N2 // 2:].contiguous()
        Wgu = tuned().prepare_gate_up(gate, up)
        act = torch.full((M, N2 // 2), float("nan"), dtype=torch.float32, device=DEV)
        tuned().gemm_swiglu(rows, Wgu, act, Rt())
        gr, ur = normed @ gate.double().T, normed @ up.double().T
        ref_act = gr / (1 + torch.exp(-gr)) * ur
        assert (act.double() - ref_act).abs().max() < 1e-2 * ref_act.abs().max()


def test_gemm_skinny_refuses_what_it_cannot_do():
    from flambeau_amd.kernels import KernelError
    from flambeau_amd.kernels.packing import pack_weight
    x, w = rnd(2, 36, dtype=torch.bfloat16), rnd(5, 36, dtype=torch.bfloat16)
    out = torch.empty(2, 5, dtype=torch.float32, device=DEV)
    with pytest.raises(KernelError, match="multiple of 8"):
        tuned().gemm_skinny(x, pack_weight(w), out)
    prepared = tuned().prepare_weight(w)
    assert prepared.packed is None                 # the dispatcher takes the plain kernel instead
    tuned().gemm(x, prepared, out)
    assert (out.double() - x.double() @ w.double().T).abs().max() < 1e-4
    with pytest.raises(KernelError, match="at most 64"):
        tuned().gemm_skinny(rnd(65, 64, dtype=torch.bfloat16), pack_weight(rnd(8, 64, dtype=torch.bfloat16)),
                            torch.empty(65, 8, dtype=torch.float32, device=DEV))
    with pytest.raises(KernelError, match="packs to"):
        tuned().gemm_skinny(rnd(2, 64, dtype=torch.bfloat16), pack_weight(rnd(8, 32, dtype=torch.bfloat16)), out)
    with pytest.raises(KernelError, match="at most 16 rows"):       # the fusions with the norm: one tile of tokens
        tuned().gemm_skinny_residual(rnd(17, 64, dtype=torch.bfloat16), pack_weight(rnd(32, 64, dtype=torch.bfloat16)),
                                     rnd(17, 32), rnd(32), torch.empty(17, 32, dtype=torch.bfloat16, device=DEV),
                                     torch.empty(17, 2, dtype=torch.float32, device=DEV), 1e-5)


# ---------------------------------------------------------------- cache, rotation, attention
def make_cache(n_pages, nkv, ps, hd, dtype):
    from flambeau_amd.kernels.ops import PagedLayerCache
    return PagedLayerCache(torch.zeros(n_pages, 2, nkv, ps, hd, dtype=dtype, device=DEV))


def read_cache(cache, table_row, t, kvh):
    """Key and value rows of token t through the block table (V is stored transposed in a page)."""
    ps, hd = cache.page_size, cache.head_dim
    page, r = int(table_row[t // ps]), t % ps
    k = cache.pool[page, 0, kvh].reshape(ps, hd)[r]
    v = cache.pool[page, 1, kvh].reshape(hd, ps)[:, r]
    return k, v


def rope_ref(x, pos, theta, rot):
    """x [n, heads, hd] double."""
    half = rot // 2
    inv = theta ** (-2.0 * torch.arange(half, dtype=torch.float64, device=x.device) / rot)
    ang = pos.double()[:, None] * inv[None]
    c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
    out = x.clone()
    lo, hi = x[..., :half], x[..., half:rot]
    out[..., :half] = lo * c - hi * s
    out[..., half:rot] = lo * s + hi * c
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,ps,rot,theta", [(4, 2, 16, 8, 16, 1e4), (6, 1, 24, 16, 24, 1e6),
                                                   (32, 8, 128, 16, 128, 1e6), (3, 3, 40, 4, 20, 5e5),
                                                   (2, 1, 64, 32, 0, 1.0)])
def test_rope_kv_write(dtype, nh, nkv, hd, ps, rot, theta):
    seqs = [(0, 5), (37, 3), (ps - 1, 2), (100, 1)]          # (start position, tokens)
    n = sum(q for _, q in seqs)
    n_pages = 96
    cache = make_cache(n_pages, nkv, ps, hd, dtype)
    perm = torch.randperm(n_pages)
    table = torch.full((len(seqs), 56), -1, dtype=torch.int32)
    used = 0
    pos, tok_seq = [], []
    for s, (st, q) in enumerate(seqs):
        nb = -(-(st + q) // ps)
        table[s, :nb] = perm[used:used + nb].int()
        used += nb
        pos += list(range(st, st + q))
        tok_seq += [s] * q
    pos_d = torch.tensor(pos, dtype=torch.int32, device=DEV)
    seq_d = torch.tensor(tok_seq, dtype=torch.int32, device=DEV)
    qkv = rnd(n, (nh + 2 * nkv) * hd, seed=13)
    q_out = torch.empty(n, nh * hd, dtype=dtype, device=DEV)
    ops().rope_kv_write(qkv, pos_d, seq_d, table.to(DEV), q_out, cache, nh, rot, theta)
    x = qkv.double()
    q_ref = x[:, :nh * hd].reshape(n, nh, hd)
    k_ref = x[:, nh * hd:(nh + nkv) * hd].reshape(n, nkv, hd)
    v_ref = x[:, (nh + nkv) * hd:].reshape(n, nkv, hd)
    if rot:
        q_ref, k_ref = rope_ref(q_ref, pos_d, theta, rot), rope_ref(k_ref, pos_d, theta, rot)
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    assert (q_out.double().reshape(n, nh, hd) - q_ref).abs().max() < tol * 4
    for i in range(n):
        for h in range(nkv):
            k, v = read_cache(cache, table[tok_seq[i]], pos[i], h)
            assert (k.double() - k_ref[i, h]).abs().max() < tol * 4
            assert (v.double() - v_ref[i, h]).abs().max() < tol * 4
    # nothing else was touched: untouched pages are still zero
    touched = set(int(p) for p in table[table >= 0])
    for p in range(n_pages):
        if p not in touched:
            assert not cache.pool[p].any()
    # the same with the angles from the step's table, and with the projection's rows in paired order
    from flambeau_amd.kernels.packing import rotary_paired_rows
    variants = []
    if rot:
        angles = torch.full((n, rot // 2, 2), float("nan"), dtype=torch.float32, device=DEV)
        ops().rope_table(pos_d, rot, theta, angles)
        variants.append(dict(table=angles))
        order = rotary_paired_rows(nh, nkv, hd, rot)
        assert (order is None) == bool(rot % 16 or hd % 16)
        if order is not None:
            assert sorted(order.tolist()) == list(range((nh + 2 * nkv) * hd))
            variants.append(dict(table=angles, paired=True, order=order))
    for v in variants:
        cache2 = make_cache(n_pages, nkv, ps, hd, dtype)
        q2 = torch.empty_like(q_out)
        order = v.pop("order", None)
        src = qkv if order is None else qkv[:, order.to(DEV)].contiguous()
        ops().rope_kv_write(src, pos_d, seq_d, table.to(DEV), q2, cache2, nh, rot, theta, **v)
        assert torch.equal(q2, q_out) and torch.equal(cache2.pool, cache.pool)


def attention_ref(q, keys, vals, pos, scale, window):
    """One query row per call site: q [nh, hd], keys/vals [T, nkv, hd] double, query at ``pos``."""
    nh, nkv = q.shape[0], keys.shape[1]
    lo = max(0, pos - window + 1) if window else 0
    out = torch.zeros_like(q)
    for h in range(nh):
        g = h // (nh // nkv)
        s = (keys[lo:pos + 1, g] @ q[h]) * scale
        p = torch.softmax(s, 0)
        out[h] = p @ vals[lo:pos + 1, g]
    return out


def build_attention_case(dtype, nh, nkv, hd, ps, seqs, seed=0):
    """Random cache contents for requests ``seqs`` = (context length, query length); the queries
    are the last ``q`` positions of each.  Returns what the kernels take and the reference."""
    torch.manual_seed(seed)
    n_pages = sum(-(-c // ps) for c, _ in seqs) + 3
    cache = make_cache(n_pages, nkv, ps, hd, dtype)
    perm = torch.randperm(n_pages)
    width = max(-(-c // ps) for c, _ in seqs) + 1
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    used = 0
    K, V = [], []
    for s, (c, _) in enumerate(seqs):
        nb = -(-c // ps)
        table[s, :nb] = perm[used:used + nb].int()
        used += nb
        k = (torch.randn(c, nkv, hd) * 0.8).to(dtype)
        v = torch.randn(c, nkv, hd).to(dtype)
        K.append(k.double().to(DEV))
        V.append(v.double().to(DEV))
        for t in range(c):
            page, r = int(table[s, t // ps]), t % ps
            cache.pool[page, 0].reshape(nkv, ps, hd)[:, r] = k[t].to(DEV)
            cache.pool[page, 1].reshape(nkv, hd, ps)[:, :, r] = v[t].to(DEV)
    pos, tok_seq = [], []
    for s, (c, ql) in enumerate(seqs):
        pos += list(range(c - ql, c))
        tok_seq += [s] * ql
    n = len(pos)
    q = (torch.randn(n, nh, hd) * 0.8).to(dtype).to(DEV)
    return dict(cache=cache, table=table.to(DEV), K=K, V=V, pos=pos, tok_seq=tok_seq, q=q, n=n,
                pos_d=torch.tensor(pos, dtype=torch.int32, device=DEV),
                seq_d=torch.tensor(tok_seq, dtype=torch.int32, device=DEV))


def attention_case_ref(case, scale, window):
    outs = []
    for i in range(case["n"]):
        s = case["tok_seq"][i]
        outs.append(attention_ref(case["q"][i].double(), case["K"][s], case["V"][s], case["pos"][i], scale, window))
    return torch.stack(outs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,ps,window", [(4, 2, 16, 8, 0), (6, 1, 24, 16, 11), (8, 2, 128, 16, 0),
                                                (5, 5, 72, 4, 30), (2, 2, 256, 32, 0), (3, 1, 10, 2, 5)])
def test_attn_plain(dtype, nh, nkv, hd, ps, window):
    seqs = [(70, 70), (33, 1), (ps * 3, 2), (1, 1), (50, 9)]
    case = build_attention_case(dtype, nh, nkv, hd, ps, seqs)
    scale = 1 / math.sqrt(hd)
    out = torch.empty(case["n"], nh * hd, dtype=dtype, device=DEV)
    ops().attn_plain(case["q"].reshape(case["n"], nh * hd), out, case["cache"], case["pos_d"], case["seq_d"],
                     case["table"], nh, scale, window)
    ref = attention_case_ref(case, scale, window)
    tol = 2e-6 if dtype == torch.float32 else 1e-2
    assert (out.double().reshape(case["n"], nh, hd) - ref).abs().max() < tol * ref.abs().max()


def test_attn_plain_refuses_large_heads():
    from flambeau_amd.kernels import KernelError
    case = build_attention_case(torch.float32, 1, 1, 8, 4, [(4, 1)])
    big = make_cache(2, 1, 4, 264, torch.float32)
    with pytest.raises(KernelError, match="head size 264"):
        ops().attn_plain(torch.zeros(1, 264, device=DEV), torch.zeros(1, 264, device=DEV), big, case["pos_d"],
                         case["seq_d"], case["table"], 1, 1.0, 0)


# ---------------------------------------------------------------- sampling
@pytest.mark.parametrize("R,V", [(1, 10), (5, 384), (3, 32768), (8, 131072), (2, 257)])
def test_argmax_first_maximum_wins(R, V):
    logits = rnd(R, V, seed=14)
    logits[0, V // 3] = 50.0
    logits[0, V - 1] = 50.0            # a later tie loses
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops().argmax(logits, out)
    want = [int(np.argmax(row)) for row in logits.cpu().numpy()]
    assert out.tolist() == want and out[0] == V // 3


@pytest.mark.parametrize("V", [97, 384, 32768])
def test_sample_is_the_inverse_cdf_in_index_order(V):
    import plain_model as pm
    R = 64
    logits = rnd(R, V, seed=15, scale=2.0)
    u = torch.rand(R, generator=torch.Generator().manual_seed(1)).to(DEV)
    u[0], u[1] = 0.0, 0.999999
    inv_t = torch.full((R,), 1 / 0.8, device=DEV)
    inv_t[2] = 0.0                                       # greedy row among the others
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops().sample(logits, inv_t, u, out)
    l, uu = logits.cpu().double().numpy(), u.cpu().double().numpy()
    assert out[2] == int(np.argmax(l[2]))
    bad = 0
    for r in range(R):
        if r == 2:
            continue
        p = np.exp((l[r] - l[r].max()) / 0.8)
        cdf = np.cumsum(p) / p.sum()
        want = int(np.searchsorted(cdf, uu[r], side="left"))
        got = int(out[r])
        if got != want:
            # a draw within rounding of a boundary may fall to the neighbour
            assert abs(got - want) == 1 and abs(cdf[min(got, want)] - uu[r]) < 1e-5
            bad += 1
    assert bad <= 2


@pytest.mark.parametrize("V", [97, 1000, 40000])
def test_penalties_and_bias_are_the_host_sampler_s(V):
    """Penalties from per-slot token counts and the bias triples against the host's rule, bit for bit:
    rows with and without a history, neutral penalties, tokens seen several times, a slot that is
    counted anew for another request, and the counts after a draw has joined them."""
    from flambeau_amd.sampling.host import penalised
    from flambeau_amd.sampling.params import SamplingParams
    rng = np.random.default_rng(V + 1)
    n_slots, R = 7, 6
    slots = [2, -1, 0, 5, 1, 3]
    params = [SamplingParams(repetition_penalty=1.7), SamplingParams(), SamplingParams(presence_penalty=0.6, frequency_penalty=0.35),
              SamplingParams(repetition_penalty=0.8, frequency_penalty=1.25), SamplingParams(),
              SamplingParams(repetition_penalty=1.3, presence_penalty=-0.4, logit_bias={1: 2.0, V - 1: -3.5, V + 5: 9.0})]
    params[1] = SamplingParams(logit_bias={0: 1.5, 17: -0.25})
    histories = [rng.integers(0, min(V, 40), int(n)).tolist() for n in (50, 0, 9, 200, 30, 0)]
    histories[3][:3] = [V - 1, V - 1, 0]
    counts = torch.randint(0, 9, (n_slots, V), dtype=torch.int16, device=DEV)       # what other requests left behind
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    f32 = lambda v: torch.tensor(np.asarray(v, dtype=np.float32), device=DEV)
    for s, h in zip(slots, histories):
        if s >= 0:
            ops().sample_history(counts, s, i32(h))
    for s, h in zip(slots, histories):
        if s >= 0:
            assert counts[s].tolist() == np.bincount(h, minlength=V).tolist()
    assert counts[4].max() > 0 and counts[6].max() > 0                                # rows nobody took are untouched
    logits = rnd(R, V, seed=21, scale=3.0)
    want = [penalised(l, p, h) for l, p, h in zip(logits.cpu().numpy(), params, histories)]

    def apply(l):
        ops().sample_penalise(l, counts, f32(slots), f32([p.repetition_penalty for p in params]),
                              f32([p.presence_penalty for p in params]), f32([p.frequency_penalty for p in params]))
        triples = [(r, t, b) for r, p in enumerate(params) if p.logit_bias for t, b in p.logit_bias.items() if t < V]
        ops().sample_bias(l, *(f32(list(c)) for c in zip(*triples)))
        return l
    got = apply(logits.clone())
    assert torch.equal(got.cpu(), torch.tensor(np.stack(want)))
    assert not torch.equal(got[0], logits[0]) and torch.equal(got[4], logits[4])
    # the drawn tokens join the histories (a row without a slot counts nowhere; a token twice in a row adds up)
    for draw in ([3, 5, 3, V - 1, 0, 8], [3, 5, 7, V - 1, 0, 8]):
        before = counts.clone()
        ops().sample_count(counts, f32(slots), i32(draw))
        for s, h, t in zip(slots, histories, draw):
            if s >= 0:
                h.append(t)
        changed = (counts != before).nonzero().tolist()
        assert sorted(changed) == sorted([s, t] for s, t in zip(slots, draw) if s >= 0)
    want = [penalised(l, p, h) for l, p, h in zip(logits.cpu().numpy(), params, histories)]
    assert torch.equal(apply(logits.clone()).cpu(), torch.tensor(np.stack(want)))
    # counts stop at 65,535
    ops().sample_history(counts, 6, i32([4] * 3))
    counts[6, 4] = -2                                                               # 65,534 as 16 bits
    for _ in range(3):
        ops().sample_count(counts, f32([6.0]), i32([4]))
    assert int(counts[6, 4]) == -1


@pytest.mark.parametrize("V", [97, 1000, 32768, 131072])
def test_filtered_sample_is_the_host_sampler_s(V):
    """Top-k, top-p and min-p on the device against the host sampler (itself checked against the plain
    one) with the same uniform numbers: rows of every combination of filters, logits with ties, rows
    without a filter and greedy rows among them (those keep what the plain kernel drew)."""
    from flambeau_amd.sampling.host import sample_host
    from flambeau_amd.sampling.params import SamplingParams
    rng = np.random.default_rng(V)
    combos = []
    for top_k in (None, 1, 5, 40, 700, 2048):
        for top_p in (None, 0.15, 0.9, 0.999, 1.0):
            for min_p in (None, 0.02, 0.6):
                combos.append((top_k, top_p, min_p))
    R = len(combos) + 2
    logits = rnd(R, V, seed=16, scale=2.5)
    logits[3] = torch.round(logits[3] * 2) / 2            # many equal logits: ties go by index
    logits[7, :] = 0.25                                    # all equal
    logits[9] = torch.round(logits[9])
    temps = rng.choice([0.6, 0.8, 1.0, 1.7], R).tolist()
    us = rng.random(R).astype(np.float32)
    us[4], us[5] = 0.0, np.float32(0.9999999)
    params = [SamplingParams(temperature=t, top_k=c[0], top_p=c[1], min_p=c[2]) for t, c in zip(temps, combos)]
    params += [SamplingParams(temperature=0.9), SamplingParams(temperature=0.0, top_k=5)]       # no filter; greedy
    assert all(p.device_ok for p in params)
    f32 = lambda v: torch.tensor(np.asarray(v, dtype=np.float32), device=DEV)
    inv_t = f32([0.0 if p.is_greedy else 1.0 / p.temperature for p in params])
    filt = [p.device_filters for p in params]
    out = torch.full((R,), -1, dtype=torch.int32, device=DEV)
    plain_draw = torch.empty(R, dtype=torch.int32, device=DEV)
    ops().sample(logits, inv_t, f32(us), plain_draw)
    out.copy_(plain_draw)
    args = (logits, inv_t, f32(us), f32([f[0] for f in filt]), f32([f[1] for f in filt]), f32([f[2] for f in filt]))
    ops().sample_filtered(*args, out)
    if V > 32768:
        # with scratch for the probabilities (formed once instead of in every pass): the same draws
        again = plain_draw.clone()
        ops().sample_filtered(*args, again, stash=torch.empty(R * V, dtype=torch.int32, device=DEV))
        assert torch.equal(again, out)
    assert out[R - 2] == plain_draw[R - 2] and out[R - 1] == plain_draw[R - 1] == int(torch.argmax(logits[R - 1]))

    class OneNumber:
        def __init__(self, u): self.u = u
        def next_f32(self): return self.u
    l = logits.cpu().numpy()
    differ = 0
    for r in range(R - 2):
        want = sample_host(l[r], params[r], [], OneNumber(us[r]))
        got = int(out[r])
        if got != want:
            # sums in another order: a draw on a boundary may fall to the neighbour in the order of probability
            p = np.exp((l[r].astype(np.float64) - l[r].max()) / temps[r]); p /= p.sum()
            order = np.argsort(-p, kind="stable").tolist()
            assert abs(order.index(got) - order.index(want)) == 1, (r, combos[r], got, want)
            differ += 1
    assert differ <= 2
    # a filter that leaves one candidate is the argmax, whatever the number drawn
    for r, c in enumerate(combos):
        if c[0] == 1:
            assert int(out[r]) == int(np.argmax(l[r]))


# ---------------------------------------------------------------- tuned attention for single rows
def decode_rows(case, picked):
    """(row, position, request, 0) of the picked rows, as the decode kernel wants them."""
    pos, seq = case["pos_d"].cpu().tolist(), case["seq_d"].cpu().tolist()
    return torch.tensor([[r, pos[r], seq[r], 0] for r in picked], dtype=torch.int32, device=DEV).reshape(-1, 4)


@pytest.mark.parametrize("n_split", [1, 2, 5])
@pytest.mark.parametrize("nh,nkv,hd,ps,window", [(32, 8, 128, 16, 0), (4, 2, 16, 8, 16), (6, 1, 24, 16, 0),
                                                (5, 5, 32, 16, 24), (20, 1, 64, 8, 0), (8, 4, 256, 32, 100),
                                                (3, 1, 40, 64, 0)])
def test_attn_decode_against_plain_and_reference(nh, nkv, hd, ps, window, n_split):
    seqs = [(700, 1), (33, 1), (ps * 3, 1), (1, 1), (257, 3), (64, 2), (32, 1), (31, 1)]
    case = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, seqs, seed=3)
    n = case["n"]
    scale = 1 / math.sqrt(hd)
    q2 = case["q"].reshape(n, nh * hd)
    rows = decode_rows(case, reversed(range(n)))      # any order of rows
    out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    hdp = -(-hd // 32) * 32
    part_o = torch.empty(n * nh * n_split * hdp, dtype=torch.float32, device=DEV)
    part_ml = torch.empty(n * nh * n_split * 2, dtype=torch.float32, device=DEV)
    tuned().attn_decode(q2, out, case["cache"], rows, case["table"], nh, scale, window, n_split, part_o, part_ml)
    plain = torch.empty_like(out)
    ops().attn_plain(q2, plain, case["cache"], case["pos_d"], case["seq_d"], case["table"], nh, scale, window)
    ref = attention_case_ref(case, scale, window)
    top = ref.abs().max()
    assert (out.double().reshape(n, nh, hd) - ref).abs().max() < 1e-2 * top
    assert (out.double() - plain.double()).abs().max() < 1.5e-2 * top


@pytest.mark.parametrize("nh,nkv,hd,ps,window", [(32, 8, 128, 16, 0), (4, 2, 16, 8, 16), (6, 1, 24, 16, 0), (20, 1, 64, 8, 0),
                                                (8, 4, 256, 32, 100), (40, 2, 32, 16, 0)])
def test_attn_decode_with_splits_per_row(nh, nkv, hd, ps, window):
    """Rows with splits of their own (long contexts many, short ones one, unused places in the list):
    the reference's result, and exactly the uniform kernel's where a row has one split."""
    seqs = [(1500, 1), (33, 1), (ps * 3, 1), (1, 1), (257, 3), (640, 2), (32, 1), (31, 1)]
    case = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, seqs, seed=9)
    n = case["n"]
    scale = 1 / math.sqrt(hd)
    q2 = case["q"].reshape(n, nh * hd)
    rows = decode_rows(case, range(n))
    per_row = tuned().decode_blocks_per_row(nh, nkv)
    items_host, firsts_host = tuned().balanced_items(rows.cpu().numpy(), per_row, window)
    splits = {int(r): int(w) >> 8 for r, _, _, w in items_host if r >= 0}
    assert len(items_host) == tuned().decode_item_budget(n, per_row) and set(splits) == set(range(n))
    assert (max(splits.values()) > 1 or 0 < window < 256) and min(splits.values()) == 1
    assert (items_host[:, 0] < 0).any() == (sum(splits.values()) < len(items_host))
    items, firsts = torch.tensor(items_host, device=DEV), torch.tensor(firsts_host, device=DEV)
    assert all(items_host[f, 0] == r and items_host[f, 3] == 256 * k for r, f, k, _ in firsts_host)
    hdp = -(-hd // 32) * 32
    part_o = torch.full((len(items_host) * nh * hdp,), float("nan"), dtype=torch.float32, device=DEV)
    part_ml = torch.full((len(items_host) * nh * 2,), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    tuned().attn_decode(q2, out, case["cache"], items, case["table"], nh, scale, window, 0, part_o, part_ml, firsts=firsts)
    ref = attention_case_ref(case, scale, window)
    assert (out.double().reshape(n, nh, hd) - ref).abs().max() < 1e-2 * ref.abs().max()
    whole = torch.empty_like(out)
    tuned().attn_decode(q2, whole, case["cache"], rows, case["table"], nh, scale, window, 1)
    one = [r for r, k in splits.items() if k == 1]
    assert torch.equal(out[one], whole[one])
    # a list with a place per row: nothing to merge, no workspace
    plain_items = rows.clone()
    plain_items[:, 3] = 256
    again = torch.full_like(out, float("nan"))
    tuned().attn_decode(q2, again, case["cache"], plain_items, case["table"], nh, scale, window, 0)
    assert torch.equal(again, whole)


def test_attn_decode_subset_of_rows_leaves_the_others_alone():
    nh, nkv, hd, ps = 8, 2, 64, 16
    case = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, [(40, 4), (90, 1)], seed=4)
    n = case["n"]
    q2 = case["q"].reshape(n, nh * hd)
    out = torch.full((n, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    tuned().attn_decode(q2, out, case["cache"], decode_rows(case, [4, 1]), case["table"], nh, 0.125, 0, 1)
    ref = attention_case_ref(case, 0.125, 0)
    assert (out[[0, 2, 3]] == 7.0).all()
    assert (out[[1, 4]].double().reshape(2, nh, hd) - ref[[1, 4]]).abs().max() < 1e-2 * ref.abs().max()


def test_attn_decode_takes_more_items_than_a_grid_has_places():
    """70,000 single rows in one call (the grid's slow index holds 65,535): all of them are computed,
    in the uniform form with two splits and with a list of items."""
    nh, nkv, hd, ps, n = 2, 1, 16, 8, 70000
    case = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, [(40, 1), (23, 1)], seed=2)
    q = (torch.randn(n, nh, hd, generator=torch.Generator().manual_seed(3)) * 0.8).to(torch.bfloat16).to(DEV)
    req = torch.arange(n, device=DEV) % 2
    pos = torch.where(req == 0, torch.arange(n, device=DEV) % 40, torch.arange(n, device=DEV) % 23)
    rows = torch.stack([torch.arange(n, device=DEV), pos, req, torch.zeros_like(req)], 1).int().contiguous()
    # the reference, all rows at once: scores against every key of the row's request, masked beyond its position
    ref = torch.zeros(n, nh, hd, dtype=torch.float64, device=DEV)
    for r in range(2):
        sel = (req == r).nonzero().squeeze(1)
        K, V = case["K"][r][:, 0], case["V"][r][:, 0]
        s = torch.einsum("nhd,td->nht", q[sel].double(), K) * 0.25
        s = s.masked_fill(torch.arange(K.shape[0], device=DEV)[None, None, :] > pos[sel][:, None, None], float("-inf"))
        ref[sel] = torch.einsum("nht,td->nhd", torch.softmax(s, -1), V)
    hdp = 32
    for n_split in (2, 0):
        out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        items = rows.clone()
        k = max(n_split, 1)
        if n_split == 0:
            items[:, 3] = 256
        part_o = torch.empty(n * nh * k * hdp, dtype=torch.float32, device=DEV)
        part_ml = torch.empty(n * nh * k * 2, dtype=torch.float32, device=DEV)
        tuned().attn_decode(q.reshape(n, nh * hd), out, case["cache"], items, case["table"], nh, 0.25, 0, n_split, part_o, part_ml)
        err = (out.double().reshape(n, nh, hd) - ref).abs().amax((1, 2))
        assert not torch.isnan(out).any() and err.max() < 1e-2 * ref.abs().max(), int(err.argmax())


# ---------------------------------------------------------------- tiled matrix product
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (65, 100, 72), (300, 250, 40), (2048, 512, 256), (129, 37, 264),
                                   (70, 4096, 4096), (200, 6144, 512), (513, 384, 96), (1000, 130, 1000)])
def test_gemm_tiled_against_plain(out_dtype, M, N, K):
    from flambeau_amd.kernels.packing import pack_weight
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=21), rnd(N, K, dtype=torch.bfloat16, seed=22, scale=0.05)
    got = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    splits = tuned().gemm_tiled_splits(M, N, K)
    ws = torch.empty(splits * M * N, dtype=torch.float32, device=DEV) if splits > 1 else None
    tuned().gemm_tiled(x, pack_weight(w), got, ws)
    ref = x.double() @ w.double().T
    scale = ref.abs().max()
    tol = 1e-5 if out_dtype == torch.float32 else 5e-3
    assert (got.double() - ref).abs().max() < tol * scale


@pytest.mark.parametrize("variant", [3, 6, 7, 8, 10])
@pytest.mark.parametrize("M,N,K", [(300, 520, 72), (129, 264, 96), (1100, 640, 256)])
def test_gemm_tiled_block_shapes(variant, M, N, K):
    """Every block shape of the tiled product (256 x 128, 192 x 128, 128 x 128, 256 x 256 and 128 x 256
    features x tokens), whichever the sizes would choose, through the plain epilogue, SwiGLU, the row scale and
    the add-to-the-stream epilogue."""
    from flambeau_amd.kernels.library import load
    from flambeau_amd.kernels.packing import pack_weight
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=23), rnd(N, K, dtype=torch.bfloat16, seed=24, scale=0.05)
    g = 1 + rnd(N, seed=25, scale=0.1)
    resid0 = rnd(M, N, seed=26)
    splits = tuned().gemm_tiled_splits(M, N, K)
    ws = torch.empty(splits * M * N, dtype=torch.float32, device=DEV) if splits > 1 else None
    got = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    tuned().gemm_tiled(x, pack_weight(w), got, ws, variant=variant)
    ref = x.double() @ w.double().T
    assert (got.double() - ref).abs().max() < 1e-5 * ref.abs().max()
    # a number of K-splits that the sizes would not choose
    ws3 = torch.empty(3 * M * N, dtype=torch.float32, device=DEV)
    got3 = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    tuned().gemm_tiled(x, pack_weight(w), got3, ws3, variant=variant, splits=3)
    assert (got3.double() - ref).abs().max() < 1e-5 * ref.abs().max()
    # gate and up rows interleaved in fours, activation in the epilogue
    inter = N // 2
    Wgu = tuned().prepare_gate_up(w[:inter].contiguous(), w[inter:2 * inter].contiguous())
    act = torch.full((M, inter), float("nan"), dtype=torch.float32, device=DEV)
    tuned().gemm_tiled(x, Wgu.packed, act, swiglu_rows=Wgu.packed_rows, variant=variant)
    want_act = torch.nn.functional.silu(ref[:, :inter]) * ref[:, inter:2 * inter]
    assert (act.double() - want_act).abs().max() < 2e-5 * want_act.abs().max()
    if splits == 1:
        resid = resid0.clone()
        xg = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ssq = torch.full((M, tuned().tiled_parts(M, N, K, variant)), float("nan"), dtype=torch.float32, device=DEV)
        rows = tuned().gemm_tiled_residual(x, pack_weight(w), resid, g, xg, ssq, 1e-5, variant=variant)
        want = resid0.double() + ref
        assert (resid.double() - want).abs().max() < 1e-5 * want.abs().max()
        assert (xg.double() - want * g.double()).abs().max() < 5e-3 * (want * g.double()).abs().max()
        assert (ssq.double().sum(dim=1) - (want * want).sum(dim=1)).abs().max() < 1e-4 * (want * want).sum(dim=1).max()
        # the rows in factors feed a product that scales by the norm itself
        w2 = rnd(200, N, dtype=torch.bfloat16, seed=27, scale=0.05)
        out2 = torch.full((M, 200), float("nan"), dtype=torch.float32, device=DEV)
        sp2 = tuned().gemm_tiled_splits(M, 200, N)
        ws2 = torch.empty(sp2 * M * 200, dtype=torch.float32, device=DEV) if sp2 > 1 else None
        tuned().gemm_tiled(rows.xg, pack_weight(w2), out2, ws2, row_scale=rows, variant=variant)
        normed = want * g.double() * torch.rsqrt((want * want).mean(dim=1, keepdim=True) + 1e-5)
        ref2 = normed @ w2.double().T
        assert (out2.double() - ref2).abs().max() < 1e-2 * ref2.abs().max()


def test_gemm_tiled_splits_k_for_small_grids():
    assert tuned().gemm_tiled_splits(2048, 4096, 4096) == 1
    assert tuned().gemm_tiled_splits(128, 4096, 4096) > 1
    from flambeau_amd.kernels import KernelError
    from flambeau_amd.kernels.packing import pack_weight
    x, w = rnd(128, 4096, dtype=torch.bfloat16), rnd(256, 4096, dtype=torch.bfloat16)
    with pytest.raises(KernelError, match="workspace"):
        tuned().gemm_tiled(x, pack_weight(w), torch.empty(128, 256, dtype=torch.float32, device=DEV))


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("waves", [0, 4, 8])
@pytest.mark.parametrize("M,N,K", [(64, 6144, 4096), (33, 4096, 14336), (17, 250, 96), (48, 37, 2048), (64, 16, 32),
                                   (20, 1000, 160), (1, 300, 64), (49, 16400, 512)])
def test_gemm_mid_against_plain(out_dtype, waves, M, N, K):
    """The kernel for 17 to 64 rows, with both block shapes and with K split or whole."""
    from flambeau_amd.kernels.library import load
    from flambeau_amd.kernels.packing import pack_weight
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=41), rnd(N, K, dtype=torch.bfloat16, seed=42, scale=0.05)
    packed = pack_weight(w)
    ref = x.double() @ w.double().T
    tol = 1e-5 if out_dtype == torch.float32 else 5e-3
    for splits in (0, 1, 3):
        n = tuned().gemm_mid_splits(M, N, K, waves, splits)
        ws = torch.full((n * M * N,), float("nan"), dtype=torch.float32, device=DEV) if n > 1 else None
        got = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
        tuned().gemm_mid(x, packed, got, ws, waves=waves, splits=splits)
        assert (got.double() - ref).abs().max() < tol * ref.abs().max(), (splits, n)


@pytest.mark.parametrize("M,H,I", [(12, 1024, 352), (16, 640, 96), (9, 5120, 64), (40, 544, 48)])
def test_gemm_mid_takes_a_row_scale_in_many_parts(M, H, I):
    """The skinny product leaves a token's sum of squares in a part per 16 features (64 to 320 parts here,
    or 34, which are not read in fours); the kernel for 17 to 64 rows, which large products use from 9 rows on, adds them
    itself before its loop: norm(resid) W^T through the factors equals the formula."""
    from flambeau_amd.kernels.packing import pack_weight
    K0 = 96
    x0, w0 = rnd(M, K0, dtype=torch.bfloat16, seed=31), rnd(H, K0, dtype=torch.bfloat16, seed=32, scale=0.1)
    g = 1 + rnd(H, seed=33, scale=0.1)
    resid = rnd(M, H, seed=34)
    want = resid.double() + x0.double() @ w0.double().T
    xg = torch.full((M, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    if M <= 16:
        ssq = torch.full((M, tuned().skinny_parts(H)), float("nan"), dtype=torch.float32, device=DEV)
        rows = tuned().gemm_skinny_residual(x0, pack_weight(w0), resid, g, xg, ssq, 1e-5)
    else:
        # any producer's parts will do: here 34 parts, which are not read in fours
        r = want.float()
        parts = torch.zeros(M, H // 16, dtype=torch.float32, device=DEV)
        for p_ in range(H // 16):
            parts[:, p_] = (r[:, p_ * 16:(p_ + 1) * 16] ** 2).sum(dim=1)
        resid.copy_(r)
        xg.copy_((r * g).to(torch.bfloat16))
        rows = tuned().NormedRows(xg, parts, 1e-5, resid, g)
    assert rows.ssq.shape[1] > 4
    normed = want * g.double() * torch.rsqrt((want * want).mean(dim=1, keepdim=True) + 1e-5)
    # plain epilogue
    w2 = rnd(200, H, dtype=torch.bfloat16, seed=35, scale=0.05)
    out = torch.full((M, 200), float("nan"), dtype=torch.float32, device=DEV)
    sp = tuned().gemm_mid_splits(M, 200, H)
    ws = torch.empty(sp * M * 200, dtype=torch.float32, device=DEV) if sp > 1 else None
    tuned().gemm_mid(rows.xg, pack_weight(w2), out, ws, row_scale=rows)
    ref = normed @ w2.double().T
    assert (out.double() - ref).abs().max() < 1e-2 * ref.abs().max()
    # gate and up with the activation in the epilogue
    Wgu = tuned().prepare_gate_up(rnd(I, H, dtype=torch.bfloat16, seed=36, scale=0.05), rnd(I, H, dtype=torch.bfloat16, seed=37, scale=0.05))
    act = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device=DEV)
    tuned().gemm_mid(rows.xg, Wgu.packed, act, swiglu_rows=Wgu.packed_rows, row_scale=rows)
    gate = normed @ rnd(I, H, dtype=torch.bfloat16, seed=36, scale=0.05).double().T
    up = normed @ rnd(I, H, dtype=torch.bfloat16, seed=37, scale=0.05).double().T
    want_act = torch.nn.functional.silu(gate) * up
    assert (act.double() - want_act).abs().max() < 2e-2 * want_act.abs().max()


def test_gemm_mid_refuses_what_it_cannot_do():
    from flambeau_amd.kernels import KernelError
    from flambeau_amd.kernels.packing import pack_weight
    out = torch.empty(20, 64, dtype=torch.float32, device=DEV)
    with pytest.raises(KernelError, match="multiple of 32"):
        tuned().gemm_mid(rnd(20, 40, dtype=torch.bfloat16), pack_weight(rnd(64, 40, dtype=torch.bfloat16)), out)
    with pytest.raises(KernelError, match="at most 64"):
        tuned().gemm_mid(rnd(65, 64, dtype=torch.bfloat16), pack_weight(rnd(64, 64, dtype=torch.bfloat16)),
                         torch.empty(65, 64, dtype=torch.float32, device=DEV))
    w = rnd(64, 4096, dtype=torch.bfloat16)
    assert tuned().gemm_mid_splits(20, 64, 4096) > 1
    with pytest.raises(KernelError, match="workspace"):
        tuned().gemm_mid(rnd(20, 4096, dtype=torch.bfloat16), pack_weight(w), out)
    # a K the kernel does not take goes to the skinny kernel through the dispatcher
    w40 = rnd(64, 40, dtype=torch.bfloat16, scale=0.1)
    x40 = rnd(20, 40, dtype=torch.bfloat16)
    tuned().gemm(x40, tuned().prepare_weight(w40), out)
    assert (out.double() - x40.double() @ w40.double().T).abs().max() < 1e-4


@pytest.mark.parametrize("M,nh,nkv,hd,rot,ps,H", [(1, 32, 8, 128, 128, 16, 4096), (8, 4, 2, 16, 16, 8, 64), (16, 5, 5, 32, 16, 16, 80),
                                                  (9, 33, 1, 144, 64, 16, 264),
                                                  (300, 6, 2, 64, 64, 16, 96), (2048, 32, 8, 128, 128, 16, 512),
                                                  (130, 3, 1, 48, 32, 32, 72), (70, 8, 8, 16, 16, 8, 40),
                                                  (64, 32, 8, 128, 128, 16, 4096), (17, 6, 2, 64, 32, 16, 96), (40, 5, 5, 32, 16, 8, 2048),
                                                  (33, 4, 2, 16, 16, 8, 40),
                                                  (512, 32, 8, 128, 128, 16, 4096), (200, 6, 2, 64, 32, 16, 4104), (96, 5, 1, 32, 16, 8, 8192)])
def test_gemm_with_rotation_and_stores_in_its_kernel(M, nh, nkv, hd, rot, ps, H):
    """The joined q/k/v projection with rows in paired order, rotated and stored by the product's own
    kernel (few rows: skinny; many rows: tiled) or, for 17 to 64 rows and for more rows whose product
    splits K, by a rotation kernel that adds the product's K-splits itself; against product + rotation
    kernel apart and float64."""
    from flambeau_amd.kernels.packing import rotary_paired_rows
    theta = 1e4
    N = (nh + 2 * nkv) * hd
    w = rnd(N, H, dtype=torch.bfloat16, seed=61, scale=0.1)
    x = rnd(M, H, dtype=torch.bfloat16, seed=62)
    order = rotary_paired_rows(nh, nkv, hd, rot).to(DEV)
    W = tuned().prepare_weight(w[order].contiguous())
    # requests of 1 to 40 tokens somewhere in their contexts, pages in a shuffled order
    torch.manual_seed(5)
    pos, seq, starts = [], [], []
    while len(pos) < M:
        k = min(int(torch.randint(1, 41, (1,))), M - len(pos))
        st = int(torch.randint(0, 200, (1,)))
        pos += range(st, st + k); seq += [len(starts)] * k; starts.append(st + k)
    width = max(-(-e // ps) for e in starts) + 1
    n_pages = sum(-(-e // ps) for e in starts) + 2
    perm = torch.randperm(n_pages).int()
    table = torch.full((len(starts), width), -1, dtype=torch.int32)
    used = 0
    for r, e in enumerate(starts):
        nb = -(-e // ps)
        table[r, :nb] = perm[used:used + nb]; used += nb
    pos_d = torch.tensor(pos, dtype=torch.int32, device=DEV)
    seq_d = torch.tensor(seq, dtype=torch.int32, device=DEV)
    table = table.to(DEV)
    angles = torch.empty(M, rot // 2, 2, dtype=torch.float32, device=DEV)
    ops().rope_table(pos_d, rot, theta, angles)
    # apart
    cache_a = make_cache(n_pages, nkv, ps, hd, torch.bfloat16)
    qkv = torch.empty(M, N, dtype=torch.float32, device=DEV)
    tuned().gemm(x, W, qkv)
    q_a = torch.empty(M, nh * hd, dtype=torch.bfloat16, device=DEV)
    ops().rope_kv_write(qkv, pos_d, seq_d, table, q_a, cache_a, nh, rot, theta, table=angles, paired=True)
    # in the product's kernel
    cache_b = make_cache(n_pages, nkv, ps, hd, torch.bfloat16)
    q_b = torch.full((M, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    store = tuned().RopeStore(pos_d, seq_d, table, angles, q_b, cache_b, nh, rot, True)
    if 16 < M <= 64 and H % 32:
        assert not tuned().gemm_rope_store(x, W, store)
        return
    split = M > 64 and tuned().gemm_tiled_splits(M, N, H) > 1
    assert split == ((M, H) in ((512, 4096), (200, 4104), (96, 8192)))          # the cases meant to split do
    assert tuned().gemm_rope_store(x, W, store)
    top = q_a.float().abs().max()
    assert (q_a.float() - q_b.float()).abs().max() <= 2e-2 * top
    assert (cache_a.pool.float() - cache_b.pool.float()).abs().max() <= 2e-2 * cache_a.pool.float().abs().max()
    assert ((cache_a.pool != 0) == (cache_b.pool != 0)).all()          # the same places were written
    if split:
        assert torch.equal(q_a, q_b) and torch.equal(cache_a.pool, cache_b.pool)      # the same sums in the same order
    elif M > 64:
        # every block shape of the tiled product writes the same
        for variant in (3, 6, 7, 8, 10):
            cache_v = make_cache(n_pages, nkv, ps, hd, torch.bfloat16)
            q_v = torch.full((M, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
            store_v = tuned().RopeStore(pos_d, seq_d, table, angles, q_v, cache_v, nh, rot, True)
            tuned().gemm_tiled_rope(x, W.packed, N, store_v, variant=variant)
            assert torch.equal(q_v, q_b) and torch.equal(cache_v.pool, cache_b.pool), variant
    # float64 reference of q
    ref = (x.double() @ w.double().T)[:, :nh * hd].reshape(M, nh, hd)
    ref = rope_ref(ref, pos_d, theta, rot)
    assert (q_b.double().reshape(M, nh, hd) - ref).abs().max() < 1.5e-2 * ref.abs().max()
    # a layer that reads another layer's cache writes none
    cache_c = make_cache(n_pages, nkv, ps, hd, torch.bfloat16)
    store_c = tuned().RopeStore(pos_d, seq_d, table, angles, torch.empty_like(q_b), cache_c, nh, rot, False)
    assert tuned().gemm_rope_store(x, W, store_c) and not cache_c.pool.any() and torch.equal(store_c.q_out, q_b)


def test_gemm_dispatch_rows_agree_across_kernels():
    """The same rows through the skinny, the middle and the tiled kernel: equal up to float rounding of sums."""
    w = rnd(512, 1024, dtype=torch.bfloat16, seed=23, scale=0.05)
    x = rnd(200, 1024, dtype=torch.bfloat16, seed=24)
    W = tuned().prepare_weight(w)
    big = torch.empty(200, 512, dtype=torch.float32, device=DEV)
    tuned().gemm(x, W, big)
    small = torch.empty(3, 512, dtype=torch.float32, device=DEV)
    tuned().gemm(x[17:20].contiguous(), W, small)
    assert (big[17:20] - small).abs().max() < 1e-5 * big.abs().max()
    middle = torch.empty(40, 512, dtype=torch.float32, device=DEV)       # the kernel for 17 to 64 rows
    tuned().gemm(x[10:50].contiguous(), W, middle)
    assert (big[10:50] - middle).abs().max() < 1e-5 * big.abs().max()


# ---------------------------------------------------------------- tiled attention for portions
def tiles_for(seqs, tile=64):
    rows, at = [], 0
    for s, (_, ql) in enumerate(seqs):
        for off in range(0, ql, tile):
            rows.append((s, at + off, min(tile, ql - off), at + off))         # every row is a row of a tile here
        at += ql
    return torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1, 4)


def split_workspace(n_rows, nh, hd, n_split):
    hdp = -(-hd // 32) * 32
    return (torch.full((n_rows * nh * n_split * hdp,), float("nan"), dtype=torch.float32, device=DEV),
            torch.full((n_rows * nh * n_split * 2,), float("nan"), dtype=torch.float32, device=DEV))


@pytest.mark.parametrize("heads_per_wave,n_split", [(0, 1), (1, 1), (0, 3), (2, 7)])
@pytest.mark.parametrize("nh,nkv,hd,ps,window", [(32, 8, 128, 16, 0), (4, 2, 16, 8, 16), (6, 1, 24, 16, 0),
                                                (5, 5, 32, 16, 24), (8, 4, 64, 8, 0), (4, 2, 256, 32, 100),
                                                (6, 3, 40, 64, 37), (2, 1, 160, 128, 0), (8, 2, 96, 16, 70)])
def test_attn_prefill_against_plain_and_reference(nh, nkv, hd, ps, window, heads_per_wave, n_split):
    # (context, queries): a whole prompt, a portion deep in a context, one that starts mid-page,
    # a portion that is no multiple of the tile, a short one
    seqs = [(200, 200), (300, 70), (ps * 5 + 3, 9), (131, 130), (64, 64), (17, 16)]
    case = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, seqs, seed=5)
    n = case["n"]
    scale = 1 / math.sqrt(hd)
    q2 = case["q"].reshape(n, nh * hd)
    out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    # with n_split > 1 the keys of every tile are split (some parts are empty: 7 parts of 1 to 5 stages) and merged
    part_o, part_ml = split_workspace(n, nh, hd, n_split) if n_split > 1 else (None, None)
    tuned().attn_prefill(q2, out, case["cache"], tiles_for(seqs), case["pos_d"], case["table"], nh, scale, window,
                         heads_per_wave, n_split=n_split, part_o=part_o, part_ml=part_ml)
    plain = torch.empty_like(out)
    ops().attn_plain(q2, plain, case["cache"], case["pos_d"], case["seq_d"], case["table"], nh, scale, window)
    ref = attention_case_ref(case, scale, window)
    top = ref.abs().max()
    err = (out.double().reshape(n, nh, hd) - ref).abs()
    assert not torch.isnan(out).any()
    assert err.max() < 1e-2 * top, f"worst at {np.unravel_index(int(err.argmax()), err.shape)}"
    assert (out.double() - plain.double()).abs().max() < 1.5e-2 * top


def test_attn_prefill_refuses_page_sizes_it_cannot_take():
    from flambeau_amd.kernels import KernelError
    for ps in (4, 12):
        case = build_attention_case(torch.bfloat16, 2, 1, 16, ps, [(20, 20)], seed=1)
        q2 = case["q"].reshape(20, 32)
        with pytest.raises(KernelError, match="power of two"):
            tuned().attn_prefill(q2, torch.empty_like(q2), case["cache"], tiles_for([(20, 20)]), case["pos_d"],
                                 case["table"], 2, 0.25, 0)
        assert not tuned().prefill_supported(case["cache"], case["table"])     # the engine takes the plain kernel


def test_attn_prefill_peaked_scores_find_single_keys():
    """One key per query is made to stand out (large q.k): the output must be that key's value
    row, wherever the key lies: first key, a page's edge, the window's first key, the query itself."""
    nh, nkv, hd, ps, window = 4, 1, 64, 16, 48
    seqs = [(160, 160)]
    case = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, seqs, seed=6)
    n = 160
    q = torch.zeros(n, nh, hd, dtype=torch.bfloat16, device=DEV)
    targets = []
    K = case["K"][0]
    for i in range(n):
        lo = max(0, i - window + 1)
        t = [lo, i, (i // ps) * ps if (i // ps) * ps >= lo else lo, min(i, lo + 15)][i % 4]
        targets.append(t)
        q[i] = (K[t, 0] / K[t, 0].norm() * 60.0).to(torch.bfloat16)          # all heads alike
    case["q"] = q
    ref = attention_case_ref(case, 1.0, window)
    for n_split in (1, 2):          # whole, and with the keys of every tile in two parts
        out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        part_o, part_ml = split_workspace(n, nh, hd, n_split) if n_split > 1 else (None, None)
        tuned().attn_prefill(q.reshape(n, nh * hd), out, case["cache"], tiles_for(seqs), case["pos_d"], case["table"], nh,
                             1.0, window, n_split=n_split, part_o=part_o, part_ml=part_ml)
        assert (out.double().reshape(n, nh, hd) - ref).abs().max() < 2e-2 * ref.abs().max()
    # and the reference indeed picks single keys
    V = case["V"][0]
    hits = sum(float((ref[i, 0] - V[targets[i], 0]).abs().max()) < 0.05 for i in range(n))
    assert hits > 0.9 * n


def build_long_attention_case(nh, nkv, hd, ps, seqs, width, seed=0):
    """``build_attention_case`` for contexts of tens of thousands of keys (bfloat16): the cache is filled
    with a few indexed copies instead of key by key, the pool starts as NaN (a key read from a page that
    was never written shows), and the block tables are ``width`` wide."""
    g = torch.Generator().manual_seed(seed)
    dtype = torch.bfloat16
    n_pages = sum(-(-c // ps) for c, _ in seqs) + 5
    from flambeau_amd.kernels.ops import PagedLayerCache
    cache = PagedLayerCache(torch.full((n_pages, 2, nkv, ps, hd), float("nan"), dtype=dtype, device=DEV))
    perm = torch.randperm(n_pages, generator=g)
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    used, K, V = 0, [], []
    for s, (c, _) in enumerate(seqs):
        nb = -(-c // ps)
        table[s, :nb] = perm[used:used + nb].int()
        used += nb
        k = (torch.randn(c, nkv, hd, generator=g) * 0.8).to(dtype).to(DEV)
        v = torch.randn(c, nkv, hd, generator=g).to(dtype).to(DEV)
        K.append(k.double())
        V.append(v.double())
        t = torch.arange(c, device=DEV)
        page, r = table[s].to(DEV)[t // ps].long(), t % ps
        keys = cache.pool[:, 0].reshape(n_pages, nkv, ps, hd)
        vals = cache.pool[:, 1].reshape(n_pages, nkv, hd, ps)
        keys[page, :, r] = k                      # [c, nkv, hd]
        vals[page, :, :, r] = v                   # values lie transposed inside a page
    pos, tok_seq = [], []
    for s, (c, ql) in enumerate(seqs):
        pos += list(range(c - ql, c))
        tok_seq += [s] * ql
    n = len(pos)
    q = (torch.randn(n, nh, hd, generator=g) * 0.8).to(dtype).to(DEV)
    return dict(cache=cache, table=table.to(DEV), K=K, V=V, pos=pos, tok_seq=tok_seq, q=q, n=n,
                pos_d=torch.tensor(pos, dtype=torch.int32, device=DEV),
                seq_d=torch.tensor(tok_seq, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("nh,nkv,hd,window", [(4, 2, 64, 0), (2, 1, 128, 0), (4, 2, 64, 5000), (2, 2, 256, 0)])
def test_attn_prefill_with_block_tables_beyond_4096_pages(nh, nkv, hd, window):
    """Portions behind 66,000 to 70,000 keys in pages of 16: block tables 8,192 wide, which a block keeps
    in LDS beside its ring (one block per compute unit then, where two fit with narrower tables).  Random
    queries against the float64 formula and the plain kernel; then queries that each single out one key
    (the first of the context, keys either side of page 4,096, the window's first key, a near one)."""
    ps, width = 16, 8192
    assert tuned().prefill_max_pages(hd) >= width
    seqs = [(70000, 72), (300, 200), (65552, 66)]
    case = build_long_attention_case(nh, nkv, hd, ps, seqs, width, seed=8)
    assert tuned().prefill_supported(case["cache"], case["table"], window)
    n = case["n"]
    scale = 1 / math.sqrt(hd)
    tiles = tiles_for(seqs)
    q2 = case["q"].reshape(n, nh * hd)
    ref = attention_case_ref(case, scale, window)
    top = ref.abs().max()
    plain = torch.empty_like(q2)
    ops().attn_plain(q2, plain, case["cache"], case["pos_d"], case["seq_d"], case["table"], nh, scale, window)
    assert (plain.double().reshape(n, nh, hd) - ref).abs().max() < 1e-2 * top
    for n_split in (1, 5, tuned().attn_prefill_splits(tiles.shape[0], nh, nkv, hd, 70000)):
        out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        part_o, part_ml = split_workspace(n, nh, hd, n_split) if n_split > 1 else (None, None)
        tuned().attn_prefill(q2, out, case["cache"], tiles, case["pos_d"], case["table"], nh, scale, window,
                             n_split=n_split, part_o=part_o, part_ml=part_ml)
        err = (out.double().reshape(n, nh, hd) - ref).abs()
        assert not torch.isnan(out).any(), n_split
        assert err.max() < 1e-2 * top, f"{n_split} splits: worst at {np.unravel_index(int(err.argmax()), err.shape)}"
        assert (out.double() - plain.double()).abs().max() < 1.5e-2 * top
    # peaked: every query of the long requests picks one key, all heads of a kv head alike
    q = case["q"].clone()
    targets = {}
    for i in range(n):
        s, p = case["tok_seq"][i], case["pos"][i]
        if seqs[s][0] < 60000:
            continue
        lo = max(0, p - window + 1) if window else 0
        t = [lo, 65535, 65536, p - 3, lo + 17, 65519][i % 6]
        t = min(max(t, lo), p)
        targets[i] = t
        for h in range(nh):
            k = case["K"][s][t, h // (nh // nkv)]
            q[i, h] = (k / k.norm() * 60.0 / scale / k.norm()).to(torch.bfloat16)       # the score of key t is 60
    case["q"] = q
    ref = attention_case_ref(case, scale, window)
    hits = sum(float((ref[i, 0] - case["V"][case["tok_seq"][i]][t, 0]).abs().max()) < 0.05 for i, t in targets.items())
    assert hits > 0.9 * len(targets)                    # the reference indeed picks single keys
    for n_split in (1, 3):
        out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        part_o, part_ml = split_workspace(n, nh, hd, n_split) if n_split > 1 else (None, None)
        tuned().attn_prefill(q.reshape(n, nh * hd), out, case["cache"], tiles, case["pos_d"], case["table"], nh, scale, window,
                             n_split=n_split, part_o=part_o, part_ml=part_ml)
        assert (out.double().reshape(n, nh, hd) - ref).abs().max() < 2e-2 * ref.abs().max(), n_split


@pytest.mark.parametrize("nh,nkv,hd,window", [(8, 8, 32, 0), (16, 8, 64, 700)])
def test_attn_prefill_grid_that_comes_in_several_rounds(nh, nkv, hd, window):
    """More blocks than the chip holds at once (over 70 tiles of 64 tokens x 8 kv heads): such a grid starts
    the tiles with the most keys first, all head groups of a tile side by side; every (tile, head group)
    must still be taken exactly once.  Three requests, so that the list of tiles is not in order of length."""
    ps = 16
    seqs = [(3000, 3000), (1500, 1300), (200, 150), (77, 77)]
    tiles = tiles_for(seqs)
    assert tiles.shape[0] * nkv > 2 * 256
    case = build_long_attention_case(nh, nkv, hd, ps, seqs, 192, seed=3)
    n = case["n"]
    scale = 1 / math.sqrt(hd)
    q2 = case["q"].reshape(n, nh * hd)
    out = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    tuned().attn_prefill(q2, out, case["cache"], tiles, case["pos_d"], case["table"], nh, scale, window)
    assert not torch.isnan(out).any()
    plain = torch.empty_like(out)
    ops().attn_plain(q2, plain, case["cache"], case["pos_d"], case["seq_d"], case["table"], nh, scale, window)
    top = plain.double().abs().max()
    assert (out.double() - plain.double()).abs().max() < 1.5e-2 * top
    # the float64 formula at the rows of a few tiles: the longest, one in the middle, the last request's
    rows = list(range(2936, 3000)) + list(range(3000 + 640, 3000 + 704)) + list(range(n - 77, n))
    for i in rows[::3]:
        s_, p_ = case["tok_seq"][i], case["pos"][i]
        ref = attention_ref(case["q"][i].double(), case["K"][s_], case["V"][s_], p_, scale, window)
        assert (out[i].double().reshape(nh, hd) - ref).abs().max() < 1e-2 * top, i


def test_attn_prefill_table_limits_come_from_the_library():
    """Tables wider than a block can keep are refused by the kernel, and the wrapper that chooses the
    kernel asks the same function; with a window only the window's pages count."""
    from flambeau_amd.kernels import KernelError
    t = tuned()
    assert t.prefill_max_pages(128) == 16384 and t.prefill_max_pages(64) == 16384 and 4096 < t.prefill_max_pages(256) < 16384
    case = build_attention_case(torch.bfloat16, 2, 1, 16, 16, [(40, 40)], seed=1)
    wide = torch.full((1, 20000), -1, dtype=torch.int32, device=DEV)
    wide[:, :case["table"].shape[1]] = case["table"]
    assert not t.prefill_supported(case["cache"], wide, 0)
    assert t.prefill_supported(case["cache"], wide, 1000)
    assert t.prefill_supported(case["cache"], wide[:, :16384].contiguous(), 0)
    q2 = case["q"].reshape(40, 32)
    with pytest.raises(KernelError, match="pages per request"):
        t.attn_prefill(q2, torch.empty_like(q2), case["cache"], tiles_for([(40, 40)]), case["pos_d"], wide, 2, 0.25, 0)
    out = torch.full_like(q2, float("nan"))
    t.attn_prefill(q2, out, case["cache"], tiles_for([(40, 40)]), case["pos_d"], wide, 2, 0.25, 24)      # a window: taken
    ref = attention_case_ref(case, 0.25, 24)
    assert (out.double().reshape(40, 2, 16) - ref).abs().max() < 1e-2 * ref.abs().max()


# ---------------------------------------------------------------- gated feed-forward in the product's epilogue
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,I,K", [(1, 14336, 4096), (8, 224, 96), (64, 136, 80), (5, 13, 40), (200, 14336, 512),
                                   (65, 160, 64), (300, 52, 72), (16, 8, 8), (40, 14336, 4096), (23, 100, 96)])
def test_gemm_swiglu_epilogue(out_dtype, M, I, K):
    gate = rnd(I, K, dtype=torch.bfloat16, seed=31, scale=0.3)
    up = rnd(I, K, dtype=torch.bfloat16, seed=32, scale=0.3)
    x = rnd(M, K, dtype=torch.bfloat16, seed=33)
    W = tuned().prepare_gate_up(gate, up)
    assert W.packed is not None and W.swiglu_cols == I and W.packed_rows % 16 == 0
    got = torch.full((M, I), float("nan"), dtype=out_dtype, device=DEV)
    if M <= 64:
        tuned().gemm_skinny(x, W.packed, got, swiglu_rows=W.packed_rows)
    else:
        tuned().gemm_tiled(x, W.packed, got, swiglu_rows=W.packed_rows)
    g, u = x.double() @ gate.double().T, x.double() @ up.double().T
    ref = g / (1 + torch.exp(-g)) * u
    tol = 2e-5 if out_dtype == torch.float32 else 6e-3
    assert (got.double() - ref).abs().max() < tol * ref.abs().max()
    if M <= 64 and K % 32 == 0:
        mid = torch.full((M, I), float("nan"), dtype=out_dtype, device=DEV)
        tuned().gemm_mid(x, W.packed, mid, swiglu_rows=W.packed_rows)
        assert (mid.double() - ref).abs().max() < tol * ref.abs().max()
