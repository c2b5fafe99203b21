"""Each kernel alone against a plain PyTorch 32-bit statement of the same operation, at sizes other
than the engine tests' (shapes taken from the reference's own kernel tests where it has them,
python/test/test_op.py and python/test/test_page_attn.py)."""
import math

import numpy as np
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu

DTYPES = [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)]   # the reference's tolerances for these dtypes


def dev():
    return torch.device("cuda:0")


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(dev())


def close(got, ref, tol):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)
    assert err <= tol, "error %.3g > %.3g" % (err, tol)


@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("T,V,H", [(32, 1000, 128), (64, 5000, 256), (127, 10000, 510), (3, 77, 88)])
def test_embedding(dtype, tol, T, V, H):
    from ginfer_amd.kernels import ops
    table = rnd((V, H), dtype, 1)
    ids = torch.randint(0, V, (T,), dtype=torch.int32, device=dev())
    ids[0], ids[-1] = V - 1, 0
    out = ops.embedding_gather(table, ids)
    assert out.dtype == torch.float32
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("T,H,eps", [(3 * 127, 128, 1e-5), (5, 1536, 1e-6), (17, 88, 3e-6), (2, 8192, 1e-6), (3, 8200, 1e-6),
                                     (4, 77, 1e-5), (2, 3584, 1e-6)])
def test_add_rmsnorm(dtype, tol, T, H, eps):
    from ginfer_amd.kernels import ops
    res = rnd((T, H), torch.float32, 2)
    delta = rnd((T, H), dtype, 3)
    gain = (1 + 0.1 * rnd((H,), torch.float32, 4)).to(dtype)
    h = res.double() + delta.double()
    ref = pm.rms_norm(h, gain.double(), eps)
    res_in = res.clone()
    out = ops.add_rmsnorm(res_in, delta, gain, eps, dtype)
    close(out, ref, tol)
    close(res_in, h, 1e-6)                                  # the residual stream took the add, in 32-bit
    # without delta: plain norm, residual untouched
    res2 = res.clone()
    out = ops.add_rmsnorm(res2, None, gain, eps, dtype)
    close(out, pm.rms_norm(res.double(), gain.double(), eps), tol)
    assert torch.equal(res2, res)
    # with rows: gathers, may name a row twice, leaves the residual alone
    rows = torch.tensor([T - 1, 0, T - 1], dtype=torch.int32, device=dev())
    res3 = res.clone()
    out = ops.add_rmsnorm(res3, delta, gain, eps, dtype, rows=rows)
    close(out, ref[rows.long()], tol)
    assert torch.equal(res3, res)
    # a 32-bit gain beside bfloat16 activations
    if dtype == torch.bfloat16:
        out = ops.add_rmsnorm(res.clone(), delta, gain.float(), eps, dtype)
        close(out, ref, tol)


@pytest.mark.parametrize("dtype,tol", DTYPES)
@pytest.mark.parametrize("T,I", [(4 * 128, 256), (2 * 511, 1024), (1023, 2048), (3, 136), (1, 8960), (5, 77), (2049, 8960)])
def test_silu_mul(dtype, tol, T, I):
    from ginfer_amd.kernels import ops
    gu = rnd((T, 2 * I), dtype, 5, scale=3.0)
    ref = torch.nn.functional.silu(gu[:, :I].double()) * gu[:, I:].double()
    close(ops.silu_mul(gu), ref, tol)
    edge = torch.tensor([[0.0, 50.0, -50.0, 1.0, 2.0, 3.0]], dtype=dtype, device=dev())
    out = ops.silu_mul(edge).float().cpu()
    assert out[0, 0] == 0 and abs(out[0, 1] - 100.0) < 1 and abs(out[0, 2]) < 1e-6


@pytest.mark.parametrize("T,I", [(8, 8), (64, 64), (72, 136), (512, 1000), (2048, 8960), (264, 24)])
def test_silu_mul_on_a_transposed_product(T, I):
    """The same activation on a product that lies transposed, [2I, T]: equal to the usual kernel on the same numbers,
    bit for bit, at sizes with whole and with broken tiles."""
    from ginfer_amd.kernels import ops
    gu = rnd((T, 2 * I), torch.bfloat16, 6, scale=3.0)
    got = ops.silu_mul_transposed(gu.t().contiguous())
    assert got.shape == (T, I) and torch.equal(got, ops.silu_mul(gu))
    ref = torch.nn.functional.silu(gu[:, :I].double()) * gu[:, I:].double()
    close(got, ref, 1e-2)
    with pytest.raises(ops.KernelError):
        ops.silu_mul_transposed(rnd((2 * 12, 16), torch.bfloat16, 1))        # I = 12 is no multiple of 8
    with pytest.raises(ops.KernelError):
        ops.silu_mul_transposed(rnd((16, 12), torch.bfloat16, 1))            # nor are 12 tokens


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 5e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("M,N,K,bias", [(2, 8, 9, True), (1031, 2000, 408, False), (512, 1024, 256, True),
                                        (130, 1001, 1000, True), (1, 1000, 128, True), (1, 197, 4216, False),
                                        (64, 64, 16, False), (65, 63, 17, True)])
def test_gemm_nt(dtype, tol, M, N, K, bias):
    from ginfer_amd.kernels import ops
    a, w = rnd((M, K), dtype, 6), rnd((N, K), dtype, 7)
    b = rnd((N,), dtype, 8) if bias else None
    ref = a.double() @ w.double().t() + (b.double() if bias else 0)
    close(ops.gemm_nt(a, w, b), ref, tol)
    if dtype == torch.bfloat16:
        out = ops.gemm_nt(a, w, b, out_dtype=torch.float32)
        assert out.dtype == torch.float32
        close(out, ref, 1e-5)


def test_gemm_nt_rows_do_not_depend_on_the_batch():
    """A row of the 32-bit product has the same bits alone and inside a larger product."""
    from ginfer_amd.kernels import ops
    a, w, b = rnd((200, 333), torch.float32, 9), rnd((129, 333), torch.float32, 10), rnd((129,), torch.float32, 11)
    full = ops.gemm_nt(a, w, b)
    for r in (0, 63, 64, 199):
        assert torch.equal(ops.gemm_nt(a[r:r + 1].contiguous(), w, b)[0], full[r])


def _fma32(a, b, c):
    """round_to_float32(a * b + c) with ONE rounding, for float32 values a, b, c: the sum is taken exactly (as a ratio
    of integers) and rounded to 24 bits, ties to even."""
    from fractions import Fraction
    exact = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
    if exact == 0:
        return np.float32(0.0)
    sign = -1 if exact < 0 else 1
    mag = abs(exact)
    e = mag.numerator.bit_length() - mag.denominator.bit_length()          # 2^e <= mag < 2^(e+2), roughly
    while Fraction(2) ** e > mag:
        e -= 1
    while Fraction(2) ** (e + 1) <= mag:
        e += 1
    e = max(e, -126)                                                       # subnormals keep the exponent of 2^-126
    scaled = mag / Fraction(2) ** (e - 23)                                 # 24 bits before the point
    q, r = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * r
    if twice > scaled.denominator or (twice == scaled.denominator and q % 2 == 1):
        q += 1
    return np.float32(sign * float(Fraction(q) * Fraction(2) ** (e - 23)))


@pytest.mark.parametrize("seed", range(30))
def test_gemm_nt_at_drawn_sizes(seed):
    """Rows, columns and K drawn at random (odd sizes, rows of a wider buffer that start at odd elements): the plain
    product, and the same bits for the same rows multiplied one, 16 and 64 at a time."""
    import random
    from ginfer_amd.kernels import ops
    rng = random.Random(700 + seed)
    M = rng.choice([1, 2, 3, 7, 8, 15, 16, 17, 33, 64, 65, 100, 129, 300])
    N = rng.choice([1, 5, 16, 17, 31, 64, 100, 130, 257, 1000])
    K = rng.choice([1, 3, 4, 8, 15, 16, 17, 31, 32, 33, 64, 100, 127, 128, 129, 500, 1536])
    dtype = rng.choice([torch.float32, torch.float32, torch.bfloat16])
    a, w = rnd((M, K), dtype, 40 + seed), rnd((N, K), dtype, 80 + seed)
    b = rnd((N,), dtype, 120 + seed) if rng.random() < 0.5 else None
    if rng.random() < 0.4:
        off = rng.choice([0, 1, 4])
        wide = torch.zeros((M, K + 8), dtype=dtype, device=a.device)
        wide[:, off:off + K] = a
        a = wide[:, off:off + K]
    full = ops.gemm_nt(a, w, b, out_dtype=torch.float32)
    close(full, a.double() @ w.double().t() + (b.double() if b is not None else 0), 5e-5)
    for rows in (1, 16, 64):
        if rows < M:
            pieces = torch.cat([ops.gemm_nt(a[r:r + rows], w, b, out_dtype=torch.float32) for r in range(0, M, rows)])
            assert torch.equal(pieces, full), "%d x %d x %d %s, %d rows at a time" % (M, N, K, dtype, rows)


@pytest.mark.parametrize("M", [3, 40, 70])
def test_gemm_nt_32_bit_is_the_chain_of_fused_multiply_adds_over_ascending_k(M):
    """What the 32-bit product IS, stated without any kernel: every element starts at zero and takes its K terms in
    ascending order, each as one fused multiply-add (one rounding); the bias is added last.  3 rows run on the
    16x16x4 matrix instruction, 40 on the same with three blocks of rows to a wavefront, 70 on the 32x32x2 matrix
    instruction: all must give these bits (the plain-FMA kernel is held against them in the test below)."""
    from ginfer_amd.kernels import ops
    N, K = 5, 37
    a, w, b = rnd((M, K), torch.float32, 31), rnd((N, K), torch.float32, 32), rnd((N,), torch.float32, 33)
    got = ops.gemm_nt(a, w, b).cpu().numpy()
    an, wn, bn = a.cpu().numpy(), w.cpu().numpy(), b.cpu().numpy()
    for m in sorted({0, 1, M // 2, M - 1}):
        for n in range(N):
            acc = np.float32(0.0)
            for k in range(K):
                acc = _fma32(an[m, k], wn[n, k], acc)
            want = np.float32(acc + bn[n])
            assert got[m, n].tobytes() == want.tobytes(), "element (%d, %d): %r, the chain gives %r" % (m, n, got[m, n], want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,bias", [(65, 130, 77, True), (200, 1536, 521, False), (128, 128, 32, True),
                                        (300, 4600, 1000, True), (2048, 1536, 1536, False), (257, 66, 3, True),
                                        (130, 66000, 40, True)])
def test_gemm_nt_on_the_matrix_cores_gives_the_bits_of_the_fma_kernel(dtype, M, N, K, bias):
    """More than 64 rows go through tiles of the 32-bit matrix-core instruction, up to 64 through a wavefront per 16
    columns with one to four blocks of 16 rows (and, from 33 rows on with 65,536 columns and more, through plain fused
    multiply-adds); all add an element's terms over ascending k into one accumulator, so the large product must equal,
    bit for bit, the same rows multiplied 64, 48, 32 and 16 at a time, and one row alone."""
    from ginfer_amd.kernels import ops
    a, w = rnd((M, K), dtype, 16), rnd((N, K), dtype, 17)
    b = rnd((N,), dtype, 18) if bias else None
    full = ops.gemm_nt(a, w, b, out_dtype=torch.float32)
    close(full, a.double() @ w.double().t() + (b.double() if bias else 0), 5e-5)
    for rows in (64, 48, 32, 16):
        pieces = torch.cat([ops.gemm_nt(a[r:r + rows].contiguous(), w, b, out_dtype=torch.float32) for r in range(0, M, rows)])
        assert torch.equal(pieces, full), "rows %d at a time: %d elements differ" % (rows, int((pieces != full).sum()))
    assert torch.equal(ops.gemm_nt(a[M - 1:].contiguous(), w, b, out_dtype=torch.float32)[0], full[M - 1])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("T,nh,nkv,hd,rd,theta", [(128, 32, 8, 128, 128, 1e4), (64, 12, 12, 64, 64, 1e4),
                                                  (9, 6, 3, 48, 48, 5e5), (5, 4, 2, 32, 16, 1e6), (7, 3, 1, 24, 20, 1e4),
                                                  (300, 12, 2, 128, 128, 1e4)])
def test_rope_and_cache_write(dtype, tol, T, nh, nkv, hd, rd, theta):
    from ginfer_amd.kernels import ops
    ps, pages = 8, 64
    qkv = rnd((T, (nh + 2 * nkv) * hd), dtype, 12)
    positions = torch.randint(0, 300, (T,), dtype=torch.int32, device=dev())
    positions[0] = 0
    sin, cos = pm.rope_tables(theta, rd, 300)
    slots = torch.randperm(pages * ps)[:T].to(torch.int64)
    slots[1] = -1 if T > 1 else slots[1]
    kp = rnd((pages, nkv, ps, hd), dtype, 13)
    vp = rnd((pages, nkv, hd, ps), dtype, 14)
    kp0, vp0 = kp.clone(), vp.clone()
    x = qkv.clone()
    ops.rope_kv_write(x, positions, cos.to(dev()), sin.to(dev()), slots.to(dev()), kp, vp, nh, nkv, hd)
    q = qkv[:, :nh * hd].double().cpu().view(T, nh, hd)
    k = qkv[:, nh * hd:(nh + nkv) * hd].double().cpu().view(T, nkv, hd)
    v = qkv[:, (nh + nkv) * hd:].cpu().view(T, nkv, hd)
    qr = pm.apply_rope(q, positions.cpu().tolist(), sin.double(), cos.double())
    kr = pm.apply_rope(k, positions.cpu().tolist(), sin.double(), cos.double())
    close(x[:, :nh * hd], qr.reshape(T, -1), tol)
    close(x[:, nh * hd:(nh + nkv) * hd], kr.reshape(T, -1), tol)
    assert torch.equal(x[:, (nh + nkv) * hd:], qkv[:, (nh + nkv) * hd:])          # v is not rotated
    assert torch.equal(x[0, :nh * hd], qkv[0, :nh * hd])                           # position 0 is the identity
    # the cache took the rotated keys and the values at the named slots, and nothing else changed
    kexp, vexp = kp0.clone().cpu(), vp0.clone().cpu()
    xk = x[:, nh * hd:(nh + nkv) * hd].cpu().view(T, nkv, hd)
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        kexp[s // ps, :, s % ps, :] = xk[t]
        vexp[s // ps, :, :, s % ps] = v[t]
    assert torch.equal(kp.cpu(), kexp) and torch.equal(vp.cpu(), vexp)
    # a run that reads another layer's cache writes nothing
    kp1, vp1 = kp0.clone(), vp0.clone()
    ops.rope_kv_write(qkv.clone(), positions, cos.to(dev()), sin.to(dev()), slots.to(dev()), kp1, vp1, nh, nkv, hd,
                      write_kv=False)
    assert torch.equal(kp1, kp0) and torch.equal(vp1, vp0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ps", [4, 8, 12, 16, 32])
@pytest.mark.parametrize("long_run", [0, 530])
def test_cache_write_of_slots_in_a_row(dtype, ps, long_run):
    """Prompt portions: tokens whose slots follow each other, starting anywhere in a page, across page ends, with
    tokens that write nothing and single tokens of other requests between them.  Every value lands in its slot of
    the transposed page and nothing else changes.  With the long run the step has tokens enough for the kernel to
    write the values of 8 tokens at a time."""
    from ginfer_amd.kernels import ops
    nh, nkv, hd, pages = 4, 2, 64, 400
    runs = [(5, 35), (-1, 1), (100, 20), (311, 1), (-1, 2), (160, 9), (330 + ps - 1, 1), (200, 17), (250, 3)]
    if long_run:
        runs.insert(3, (701, long_run))
    slots = []
    for first, n in runs:
        slots += [-1] * n if first < 0 else list(range(first, first + n))
    assert len(set(x for x in slots if x >= 0)) == sum(1 for x in slots if x >= 0) and max(slots) < pages * ps
    T = len(slots)
    slots = torch.tensor(slots, dtype=torch.int64)
    qkv = rnd((T, (nh + 2 * nkv) * hd), dtype, 21)
    positions = torch.arange(T, dtype=torch.int32, device=dev())
    sin, cos = pm.rope_tables(1e4, hd, T)
    kp, vp = rnd((pages, nkv, ps, hd), dtype, 22), rnd((pages, nkv, hd, ps), dtype, 23)
    kexp, vexp = kp.clone().cpu(), vp.clone().cpu()
    x = qkv.clone()
    ops.rope_kv_write(x, positions, cos.to(dev()), sin.to(dev()), slots.to(dev()), kp, vp, nh, nkv, hd)
    xk = x[:, nh * hd:(nh + nkv) * hd].cpu().view(T, nkv, hd)
    v = qkv[:, (nh + nkv) * hd:].cpu().view(T, nkv, hd)
    for t in range(T):
        sl = int(slots[t])
        if sl >= 0:
            kexp[sl // ps, :, sl % ps, :] = xk[t]
            vexp[sl // ps, :, :, sl % ps] = v[t]
    assert torch.equal(kp.cpu(), kexp) and torch.equal(vp.cpu(), vexp)
    # the rotation is the one of single tokens
    one = qkv[40:41].clone()
    ops.rope_kv_write(one, positions[40:41].contiguous(), cos.to(dev()), sin.to(dev()), slots[40:41].to(dev()),
                      kp.clone(), vp.clone(), nh, nkv, hd)
    assert torch.equal(one[0], x[40])


# ----------------------------------------------------------------------------- attention

def _paged_case(seqs, nh, nkv, hd, ps, dtype, seed, window=None, spike=None):
    """seqs: list of (q_len, kv_len).  Builds a scrambled paged cache (pages in random order, unused
    slots filled with NaN) and the step's arrays; returns the operands and the plain result."""
    g = torch.Generator().manual_seed(seed)
    E = len(seqs)
    blocks = [-(-kv // ps) for _, kv in seqs]
    num_pages = sum(blocks) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    width = max(blocks) + 1
    bt = torch.full((E, width), -1, dtype=torch.int32)
    kp = torch.full((num_pages, nkv, ps, hd), float("nan"))
    vp = torch.full((num_pages, nkv, hd, ps), float("nan"))
    T = sum(q for q, _ in seqs)
    q = torch.randn((T, nh, hd), generator=g)
    ent, pos = [], []
    refs = []
    o = 0
    for e, (ql, kv) in enumerate(seqs):
        k = torch.randn((kv, nkv, hd), generator=g)
        v = torch.randn((kv, nkv, hd), generator=g)
        qpos = list(range(kv - ql, kv))
        if spike is not None:
            # one far key that the last query of the request must find: its score stands out
            c = spike(e, ql, kv)
            if c is not None:
                k[c, :, :] = 0
                k[c, :, 0] = 40.0
                q[o + ql - 1, :, :] = 0
                q[o + ql - 1, :, 0] = math.sqrt(hd)       # score 40 at key c, about N(0, 1) elsewhere
                v[c, :, :] = 7.0
        k, v, = k.to(dtype).float(), v.to(dtype).float()
        pages = [perm.pop() for _ in range(blocks[e])]
        bt[e, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        for c in range(kv):
            kp[pages[c // ps], :, c % ps, :] = k[c]
            vp[pages[c // ps], :, :, c % ps] = v[c]
        qe = q[o:o + ql].to(dtype).float()
        refs.append(pm.attention(qe.double(), k.double(), v.double(), qpos, window))
        ent += [e] * ql
        pos += qpos
        o += ql
    d = dev()
    ops_in = dict(q=q.to(dtype).reshape(T, nh * hd).to(d), k_pages=kp.to(dtype).to(d), v_pages=vp.to(dtype).to(d),
                  block_table=bt.to(d), token_entry=torch.tensor(ent, dtype=torch.int32, device=d),
                  positions=torch.tensor(pos, dtype=torch.int32, device=d))
    return ops_in, torch.cat(refs).reshape(T, nh * hd), seqs


ATTN_HEADS = [(32, 8, 128), (12, 12, 64), (12, 2, 128), (6, 1, 32), (4, 2, 16), (6, 3, 48), (5, 5, 80)]
ATTN_SEQS = [[(1, 128), (1, 256)], [(64, 64), (128, 128)], [(1, 500), (9, 9)], [(125, 260), (63, 63)],
             [(1, 1), (2, 2), (1, 17), (33, 40)], [(1, 1280), (1, 2561)]]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("nh,nkv,hd", ATTN_HEADS)
@pytest.mark.parametrize("seqs", ATTN_SEQS)
def test_paged_attention_generic(dtype, tol, nh, nkv, hd, seqs):
    from ginfer_amd.kernels import ops
    if sum(kv for _, kv in seqs) * nkv * hd > 3e6:
        if (nh, nkv, hd) not in ((12, 2, 128), (6, 1, 32)):
            pytest.skip("large case kept for two head shapes")
    for ps in (16, 8) if hd <= 48 else (16,):
        a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, dtype, seed=hd + ps)
        out = ops.paged_attention_generic(a["q"], a["k_pages"], a["v_pages"], a["block_table"], a["token_entry"],
                                          a["positions"], nh, nkv, hd, 1.0 / math.sqrt(hd))
        close(out, ref, tol)


@pytest.mark.parametrize("seed", range(24))
def test_paged_attention_generic_at_drawn_sizes_whatever_shares_a_workgroup(seed):
    """Head layouts, head sizes, page sizes, windows and mixes of requests drawn at random, in 32-bit: the plain result,
    and the same bits whether a workgroup holds one token, two, or what the library chooses (which also decides whether
    the loading wavefronts and the second tile buffer of a step with few workgroups are used)."""
    import random
    from ginfer_amd.kernels import ops
    rng = random.Random(300 + seed)
    nkv, group = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 6, 7, 8])
    nh, hd, ps = nkv * group, rng.choice([16, 24, 32, 48, 64, 80, 128]), rng.choice([4, 8, 16, 32])
    window = rng.choice([None, None, None, 5, 40, 100])
    kind = rng.choice(["single tokens", "portions and single tokens", "a prompt"])
    if kind == "single tokens":
        seqs = [(1, rng.randint(1, 300)) for _ in range(rng.randint(1, 6))]
    elif kind == "a prompt":
        n = rng.randint(2, 120)
        seqs = [(n, n + rng.choice([0, 0, 17, 64]))]
    else:
        seqs = [(ql, ql + rng.randint(0, 150)) for ql in (rng.choice([1, 1, 2, 5, 33]) for _ in range(rng.randint(2, 5)))]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.float32, seed=seed, window=window)
    outs = [ops.paged_attention_generic(a["q"], a["k_pages"], a["v_pages"], a["block_table"], a["token_entry"],
                                        a["positions"], nh, nkv, hd, 1.0 / math.sqrt(hd), window=window,
                                        tokens_per_workgroup=tq) for tq in (0, 1, 2)]
    close(outs[0], ref, 1e-5)
    what = "%s %s, %d heads in %d groups of size %d, pages of %d, window %s" % (kind, seqs, nh, nkv, hd, ps, window)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), what


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("seed", range(24))
def test_paged_attention_on_the_matrix_cores_gives_the_bits_of_the_wavefront_per_token(dtype, tol, seed):
    """Steps of 32 tokens and more that hold prompt portions, at head sizes in steps of 16 up to 128, run on the matrix
    cores when the library chooses (tokens_per_workgroup 0): a wavefront per head and 16 tokens; with one token to a
    workgroup the heads of a kv group are the columns of the matrix cores' products (where pages allow 16-byte loads);
    with two, a wavefront per (token, head) without the matrix cores.  All add a score's products over ascending
    dimensions and an output's over ascending keys as fused multiply-adds, so they give the same bits: portions of several requests in one group of 32 tokens, single tokens
    between them (runs of fewer than 8 tokens are left to the wavefronts per token in the same call), windows, kv groups
    that do not fill a workgroup, pages smaller than a load."""
    import random
    from ginfer_amd.kernels import ops
    rng = random.Random(900 + seed)
    nkv, group = rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 6, 7, 8, 12])
    nh, hd, ps = nkv * group, (16, 32, 48, 64, 80, 96, 112, 128)[seed % 8], rng.choice([2, 4, 8, 16, 32, 64])
    window = rng.choice([None, None, 7, 40, 100, 130])
    kind = rng.choice(["a prompt", "portions", "portions and single tokens"])
    if kind == "a prompt":
        n = rng.randint(32, 300)
        seqs = [(n, n + rng.choice([0, 0, 17, 64, 200]))]
    elif kind == "portions":
        seqs = [(ql, ql + rng.randint(0, 200)) for ql in (rng.choice([2, 5, 20, 33, 64, 90]) for _ in range(rng.randint(2, 4)))]
    else:
        seqs = [(ql, ql + rng.randint(0, 200)) for ql in (rng.choice([1, 1, 1, 2, 7, 8, 9, 30, 45]) for _ in range(rng.randint(3, 7)))]
    # enough tokens that the library does not give the whole step to the kernel for single tokens (it does up to 512
    # workgroups of a token and a kv head)
    while sum(ql for ql, _ in seqs) * nkv <= 512:
        seqs.append((rng.choice([16, 64, 150]), rng.choice([16, 64, 150]) + rng.randint(0, 100)))
    seqs = [(ql, max(ql, kv)) for ql, kv in seqs]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, dtype, seed=seed, window=window)
    outs = [ops.paged_attention_generic(a["q"], a["k_pages"], a["v_pages"], a["block_table"], a["token_entry"],
                                        a["positions"], nh, nkv, hd, 1.0 / math.sqrt(hd), window=window,
                                        tokens_per_workgroup=tq) for tq in (0, 1, 2)]
    what = "%s %s, %d heads in %d groups of size %d, pages of %d, window %s" % (kind, seqs, nh, nkv, hd, ps, window)
    close(outs[0], ref, tol)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), what
    if min(ql for ql, _ in seqs) >= 8:                # the caller may then say so, and the second kernel is left out
        alone = ops.paged_attention_generic(a["q"], a["k_pages"], a["v_pages"], a["block_table"], a["token_entry"],
                                            a["positions"], nh, nkv, hd, 1.0 / math.sqrt(hd), window=window,
                                            tokens_per_workgroup=-1)
        assert torch.equal(alone, outs[1]), what


@pytest.mark.parametrize("seqs,window", [([(2048, 2048)], None), ([(1, 900), (1500, 2100), (1, 64), (3, 700), (540, 540)], None),
                                         ([(1100, 1700)], 600)])
def test_paged_attention_on_the_matrix_cores_at_the_sizes_of_the_benchmark(seqs, window):
    """The 32-bit attention at the 1.5B shape's heads (12 in 2 groups of size 128, pages of 16): a 2,048-token prompt, a
    step that mixes long portions with single tokens, and a window; against the plain result, and the same bits from
    the matrix cores and from a wavefront per token."""
    from ginfer_amd.kernels import ops
    nh, nkv, hd, ps = 12, 2, 128, 16
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.float32, seed=11, window=window)
    outs = [ops.paged_attention_generic(a["q"], a["k_pages"], a["v_pages"], a["block_table"], a["token_entry"],
                                        a["positions"], nh, nkv, hd, 1.0 / math.sqrt(hd), window=window,
                                        tokens_per_workgroup=tq) for tq in (0, 1, 2)]
    close(outs[0], ref, 1e-5)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("window", [1, 5, 16, 40, 64, 100])
def test_paged_attention_window(dtype, tol, window):
    from ginfer_amd.kernels import ops
    nh, nkv, hd, ps = 6, 3, 48, 16
    seqs = [(1, 200), (30, 90), (7, 7), (1, window), (1, window + 1), (50, 130)]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, dtype, seed=window, window=window)
    out = ops.paged_attention_generic(a["q"], a["k_pages"], a["v_pages"], a["block_table"], a["token_entry"],
                                      a["positions"], nh, nkv, hd, 1.0 / math.sqrt(hd), window=window)
    close(out, ref, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("where", ["first", "page_edge", "before_page_edge", "tile_edge", "last", "window_edge",
                                   "behind_window"])
def test_paged_attention_finds_one_far_key(dtype, where):
    """Random keys hide a skipped key among hundreds; here one key carries nearly all the weight, so
    the output is that key's value (7) if and only if the kernel reads it."""
    from ginfer_amd.kernels import ops
    nh, nkv, hd, ps = 4, 2, 32, 16
    kv = 300
    window = 100 if "window" in where else None
    place = {"first": 0, "page_edge": 16 * 9, "before_page_edge": 16 * 9 - 1, "tile_edge": 64 * 3, "last": kv - 1,
             "window_edge": kv - 100, "behind_window": kv - 101}[where]
    seqs = [(1, kv), (20, kv)]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, dtype, seed=5, window=window, spike=lambda e, ql, n: place)
    out = ops.paged_attention_generic(a["q"], a["k_pages"], a["v_pages"], a["block_table"], a["token_entry"],
                                      a["positions"], nh, nkv, hd, 1.0 / math.sqrt(hd), window=window)
    close(out, ref, 1e-5 if dtype == torch.float32 else 2e-2)
    last_rows = out.float().cpu()[[0, 20]]
    if where == "behind_window":
        assert (last_rows.abs() < 3).all()
    else:
        assert (last_rows - 7.0).abs().max() < 0.1


@pytest.mark.parametrize("R,V", [(1, 128), (1, 1024), (1, 4096), (2, 128), (17, 1024), (33, 4096), (3, 777), (2, 151936)])
def test_argmax_lowest_index(R, V):
    from ginfer_amd.kernels import ops
    x = rnd((R, V), torch.float32, 20)
    out = ops.sample_rows(x).cpu().numpy()
    assert (out == np.argmax(x.cpu().numpy(), axis=1)).all()
    # ties: the lowest index wins, wherever the equal values lie
    y = torch.zeros((3, V), device=dev())
    y[1, V - 1] = y[1, V // 2] = 5.0
    y[2, V // 3] = y[2, V // 3 + 1] = 2.0
    assert ops.sample_rows(y).cpu().tolist() == [0, V // 2, V // 3]


@pytest.mark.parametrize("V", [777, 4096, 151936])
def test_temperature_sampling(V):
    from ginfer_amd.kernels import ops
    R = 64
    x = rnd((R, V), torch.float32, 21, scale=2.0)
    temps = torch.full((R,), 0.8, device=dev())
    temps[::7] = 0.0
    g = torch.Generator().manual_seed(3)
    uni = torch.rand((R,), generator=g).to(dev())
    out = ops.sample_rows(x, temps, uni).cpu().tolist()
    agree = 0
    for r in range(R):
        agree += int(out[r] == pm.sample_token(x[r].cpu(), float(temps[r]), float(uni[r])))
    assert agree >= R - 1, "%d of %d draws agree with the plain sampler" % (agree, R)
    # temperature -> 0 tends to the argmax
    cold = ops.sample_rows(x, torch.full((R,), 1e-4, device=dev()), uni).cpu().tolist()
    assert cold == x.argmax(dim=1).cpu().tolist()
    # uniform number 0 picks the first token with mass; just below 1 the last
    one = torch.zeros((1, V), device=dev())
    assert ops.sample_rows(one, torch.ones(1, device=dev()), torch.zeros(1, device=dev())).item() == 0
    assert ops.sample_rows(one, torch.ones(1, device=dev()), torch.full((1,), 0.9999999, device=dev())).item() == V - 1


@pytest.mark.parametrize("V", [777, 5000, 151936])
def test_sampling_does_not_depend_on_the_rows_beside(V):
    """A row's token is a function of its logits, temperature and uniform number alone: the same row drawn alone,
    among 7 and among 300 rows gives the same token, bit for bit in the sums behind it."""
    from ginfer_amd.kernels import ops
    R = 300
    x = rnd((R, V), torch.float32, 33, scale=3.0)
    temps = torch.full((R,), 1.3, device=dev())
    temps[::5] = 0.0
    uni = torch.rand((R,), generator=torch.Generator().manual_seed(4)).to(dev())
    every = ops.sample_rows(x, temps, uni).cpu().tolist()
    some = ops.sample_rows(x[10:17], temps[10:17].contiguous(), uni[10:17].contiguous()).cpu().tolist()
    assert some == every[10:17]
    for r in (0, 1, 151, 299):
        assert ops.sample_rows(x[r:r + 1], temps[r:r + 1].contiguous(), uni[r:r + 1].contiguous()).item() == every[r]


def test_kernels_refuse_what_they_cannot_take():
    from ginfer_amd.kernels import ops, KernelError
    with pytest.raises(KernelError):
        ops.gemm_nt(rnd((4, 8), torch.float32, 1), rnd((4, 9), torch.float32, 2))
    with pytest.raises(KernelError):
        ops.add_rmsnorm(rnd((4, 8), torch.float32, 1), rnd((4, 9), torch.float32, 2), rnd((8,), torch.float32, 3), 1e-6,
                        torch.float32)
    with pytest.raises(KernelError):
        ops.embedding_gather(rnd((10, 8), torch.float32, 1), torch.zeros(3, dtype=torch.int64, device=dev()))
    with pytest.raises(KernelError):
        ops.silu_mul(rnd((4, 7), torch.float32, 1))
    with pytest.raises(KernelError):
        ops.add_rmsnorm(torch.zeros(4, 8), None, torch.ones(8), 1e-6, torch.float32)      # CPU tensors


# ----------------------------------------------------------------------------- matrix-core attention

class _Step:
    """The few fields of a step that the attention dispatcher reads."""

    def __init__(self, seqs, a):
        self.num_entries = len(seqs)
        self.host_q_len = [q for q, _ in seqs]
        self.host_q_start = [kv - q for q, kv in seqs]
        self.token_entry, self.positions = a["token_entry"], a["positions"]
        self.extra = {}


MFMA_SEQS = ATTN_SEQS + [[(1, 31), (1, 32), (1, 33), (1, 64), (1, 65)], [(31, 31), (33, 95), (2, 2), (17, 100)],
                         [(1, 5000)], [(300, 700)]]


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("nh,nkv,hd", ATTN_HEADS + [(40, 2, 64), (3, 1, 256), (18, 1, 16), (7, 1, 64), (8, 4, 256)])
@pytest.mark.parametrize("seqs", MFMA_SEQS)
def test_paged_attention_mfma(nh, nkv, hd, seqs, wide, monkeypatch):
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)    # 32 or 16 rows to a wavefront
    if wide and max(q for q, _ in seqs) == 1:
        pytest.skip("no prompt rows in this case")
    if sum(kv for _, kv in seqs) * nkv * hd > 3e6 and (nh, nkv, hd) not in ((12, 2, 128), (6, 1, 32)):
        pytest.skip("large case kept for two head shapes")
    for ps in (16, 8, 64) if hd <= 48 else (16,):
        a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.bfloat16, seed=hd + ps)
        out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a), nh, nkv, hd,
                                       1.0 / math.sqrt(hd))
        close(out, ref, 2e-2)


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("nh,nkv,hd", [(12, 2, 128), (28, 4, 128), (6, 3, 64), (14, 2, 64), (4, 2, 256), (6, 1, 256), (9, 3, 128),
                                       (8, 2, 128), (5, 1, 64), (12, 2, 48)])
@pytest.mark.parametrize("seqs", [[(300, 700)], [(31, 31), (33, 95), (2, 2), (17, 100)], [(125, 260), (63, 63), (1, 40)],
                                  [(64, 64), (128, 128)], [(257, 1300)]])
def test_paged_attention_mfma_heads_side_by_side(nh, nkv, hd, seqs, wide, monkeypatch):
    """The prefill kernel that shares keys and values among the heads of a kv group through LDS runs where a step
    has tiles enough to fill the chip; here it is made to run on small cases too (every head size it is built for,
    groups of 2 to 7 heads with one or two streams of tiles, page sizes of 8 to 64, portions that start inside a
    sequence), beside a head size that it is not built for."""
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)
    monkeypatch.setattr(ops.TUNING, "prefill_fill_workgroups", 1)
    for ps in (16, 8, 32, 64):
        a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.bfloat16, seed=hd + ps)
        out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a), nh, nkv, hd,
                                       1.0 / math.sqrt(hd))
        close(out, ref, 2e-2)


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("window", [1, 5, 16, 40, 64, 100])
def test_paged_attention_mfma_heads_side_by_side_window(window, wide, monkeypatch):
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)
    monkeypatch.setattr(ops.TUNING, "prefill_fill_workgroups", 1)
    nh, nkv, hd = 6, 2, 64
    seqs = [(30, 90), (7, 7), (50, 130), (200, 330), (1, 2000)]
    for ps in (16, 8):
        a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.bfloat16, seed=window, window=window)
        out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a), nh, nkv, hd,
                                       1.0 / math.sqrt(hd), window=window)
        close(out, ref, 2e-2)


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("where", ["first", "page_edge", "before_page_edge", "tile_edge", "before_tile_edge", "split_edge",
                                   "last", "window_edge", "behind_window"])
def test_paged_attention_mfma_heads_side_by_side_finds_one_far_key(where, wide, monkeypatch):
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)
    monkeypatch.setattr(ops.TUNING, "prefill_fill_workgroups", 1)
    nh, nkv, hd, ps = 6, 2, 64, 16
    kv = 300
    window = 100 if "window" in where else None
    place = {"first": 0, "page_edge": 16 * 9, "before_page_edge": 16 * 9 - 1, "tile_edge": 32 * 3, "before_tile_edge": 95,
             "split_edge": 64, "last": kv - 1, "window_edge": kv - 100, "behind_window": kv - 101}[where]
    seqs = [(20, kv), (40, kv)]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.bfloat16, seed=5, window=window, spike=lambda e, ql, n: place)
    out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a), nh, nkv, hd,
                                   1.0 / math.sqrt(hd), window=window)
    close(out, ref, 2e-2)
    last_rows = out.float().cpu()[[19, 59]]
    if where == "behind_window":
        assert (last_rows.abs() < 3).all()
    else:
        assert (last_rows - 7.0).abs().max() < 0.1


def _force_key_parts(monkeypatch, ops, share):
    """Makes the dispatcher deal the keys of every tile that has more than `share` tiles of 32 keys to several workgroups,
    whatever the step's size (the rule itself looks for a short prompt alone in a step)."""
    real = ops.key_parts
    monkeypatch.setattr(ops.TUNING, "prefill_split_max_workgroups", 1 << 30)
    monkeypatch.setattr(ops.TUNING, "prefill_split_min_key_tiles", 0)
    monkeypatch.setattr(ops.TUNING, "prefill_split_imbalance", 1e-9)
    units = {}
    monkeypatch.setattr(ops, "key_parts", lambda tiles, tile_rows, window, wgs, streams, compute_units=256:
                        real(tiles, tile_rows, window, wgs, streams,
                             compute_units=max(1, int(units.setdefault("n", sum((t[3] + t[2] - 1) // 32 + 1 for t in tiles) * wgs / share)))))


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("shared", [False, True])
@pytest.mark.parametrize("nh,nkv,hd", [(12, 2, 128), (6, 3, 64), (6, 1, 48), (4, 2, 256), (5, 1, 80)])
@pytest.mark.parametrize("seqs,window,share", [([(300, 700)], None, 5), ([(257, 1300), (40, 40), (1, 90)], None, 9),
                                               ([(200, 330), (64, 64)], 100, 2), ([(150, 150)], None, 1.5),
                                               ([(96, 2100)], None, 30)])
def test_paged_attention_mfma_keys_in_parts(nh, nkv, hd, seqs, window, share, shared, wide, monkeypatch):
    """The keys of the heaviest prompt tiles dealt to several workgroups, merged by the kernel that merges the splits of
    single tokens: forced here at small sizes, for the kernel that keeps its operands in registers and the one that
    shares them through LDS, beside tiles that stay whole and single tokens; up to eight parts."""
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)
    monkeypatch.setattr(ops.TUNING, "prefill_fill_workgroups", 1 if shared else 1 << 30)
    _force_key_parts(monkeypatch, ops, share)
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, 16, torch.bfloat16, seed=hd + len(seqs), window=window)
    step = _Step(seqs, a)
    out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], step, nh, nkv, hd,
                                   1.0 / math.sqrt(hd), window=window)
    plans = [v for k, v in step.extra.items() if k[0] == "attention_plan"]
    assert plans and plans[0]["n_part_rows"] > 0 and plans[0]["num_parts"] >= 2, "the keys were not dealt out"
    close(out, ref, 2e-2)


@pytest.mark.parametrize("where", ["first", "part_edge", "before_part_edge", "last"])
def test_paged_attention_mfma_keys_in_parts_finds_one_far_key(where, monkeypatch):
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0)
    monkeypatch.setattr(ops.TUNING, "prefill_fill_workgroups", 1)
    _force_key_parts(monkeypatch, ops, 6)
    nh, nkv, hd, ps, kv = 6, 2, 64, 16, 640
    seqs = [(40, kv)]
    # with a share of 6 tiles the 20 tiles of 32 keys fall into 4 parts of 6 (rounded to the workgroup's streams): edges at 192, 384, 576
    place = {"first": 0, "part_edge": 384, "before_part_edge": 383, "last": kv - 1}[where]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.bfloat16, seed=5, spike=lambda e, ql, n: place)
    step = _Step(seqs, a)
    out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], step, nh, nkv, hd, 1.0 / math.sqrt(hd))
    plan = [v for k, v in step.extra.items() if k[0] == "attention_plan"][0]
    assert plan["num_parts"] >= 3
    close(out, ref, 2e-2)
    assert (out.float().cpu()[39] - 7.0).abs().max() < 0.1


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("hd", list(range(16, 257, 16)))
def test_paged_attention_mfma_every_head_size(hd, wide, monkeypatch):
    """Head sizes in steps of 16 up to 256, each with a group of 3 heads: portions of prompts beside single tokens."""
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)
    seqs = [(1, 130), (37, 101), (64, 64), (1, 17), (2, 300)]
    a, ref, _ = _paged_case(seqs, 6, 2, hd, 16, torch.bfloat16, seed=hd)
    out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a), 6, 2, hd,
                                   1.0 / math.sqrt(hd))
    close(out, ref, 2e-2)


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("window", [1, 5, 16, 40, 64, 100])
def test_paged_attention_mfma_window(window, wide, monkeypatch):
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)
    nh, nkv, hd, ps = 6, 3, 48, 16
    seqs = [(1, 200), (30, 90), (7, 7), (1, window), (1, window + 1), (50, 130), (1, 2000)]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.bfloat16, seed=window, window=window)
    out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a), nh, nkv, hd,
                                   1.0 / math.sqrt(hd), window=window)
    close(out, ref, 2e-2)


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("where", ["first", "page_edge", "before_page_edge", "tile_edge", "before_tile_edge", "split_edge",
                                   "last", "window_edge", "behind_window"])
def test_paged_attention_mfma_finds_one_far_key(where, wide, monkeypatch):
    from ginfer_amd.kernels import ops
    monkeypatch.setattr(ops.TUNING, "prefill_wide_tiles_from", 0 if wide else 1 << 30)
    nh, nkv, hd, ps = 4, 2, 32, 16
    kv = 300
    window = 100 if "window" in where else None
    place = {"first": 0, "page_edge": 16 * 9, "before_page_edge": 16 * 9 - 1, "tile_edge": 32 * 3, "before_tile_edge": 95,
             "split_edge": 64, "last": kv - 1, "window_edge": kv - 100, "behind_window": kv - 101}[where]
    seqs = [(1, kv), (20, kv)]
    a, ref, _ = _paged_case(seqs, nh, nkv, hd, ps, torch.bfloat16, seed=5, window=window, spike=lambda e, ql, n: place)
    out = ops.paged_attention_mfma(a["q"], a["k_pages"], a["v_pages"], a["block_table"], _Step(seqs, a), nh, nkv, hd,
                                   1.0 / math.sqrt(hd), window=window)
    close(out, ref, 2e-2)
    last_rows = out.float().cpu()[[0, 20]]
    if where == "behind_window":
        assert (last_rows.abs() < 3).all()
    else:
        assert (last_rows - 7.0).abs().max() < 0.1


@pytest.mark.parametrize("M", [1, 2, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K,bias", [(2048, 1536, True), (1536, 1536, False), (17920, 1536, False), (1536, 8960, False),
                                      (1000, 192, True), (197, 4216, False), (33, 8, True), (777, 88, False), (5000, 72, True),
                                      # from 16,384 columns on, up to 16 rows: dealt evenly to a multiple of 256 workgroups
                                      (20000, 72, True), (40010, 40, True), (16390, 200, False)])
def test_gemm_skinny(M, N, K, bias):
    from ginfer_amd.kernels import ops
    a, w = rnd((M, K), torch.bfloat16, 30), rnd((N, K), torch.bfloat16, 31)
    b = rnd((N,), torch.bfloat16, 32) if bias else None
    assert ops.gemm_skinny_supported(a, w)
    ref = a.double() @ w.double().t() + (b.double() if bias else 0)
    close(ops.gemm_skinny(a, w, b), ref, 1e-2)
    out = ops.gemm_skinny(a, w, b, out_dtype=torch.float32)
    assert out.dtype == torch.float32
    close(out, ref, 1e-5)
    # a row does not depend on how many rows stand beside it: bit for bit among products of the same tiling
    # (packed tiles, for up to 8 rows, add the halves of K up separately), to rounding across tilings
    if M > 1:
        for pack in (1, 2) if M <= 8 else (1,):
            both = ops.gemm_skinny(a, w, b, out_dtype=torch.float32, pack=pack)
            one = ops.gemm_skinny(a[M - 1:M], w, b, out_dtype=torch.float32, pack=pack)
            assert torch.equal(one[0], both[M - 1])
        close(ops.gemm_skinny(a[M - 1:M], w, b, out_dtype=torch.float32)[0], out[M - 1], 1e-6)
    # rows of a wider buffer (a view with a row stride), as the fused projections hand them on
    wide = rnd((M, K + 64), torch.bfloat16, 33)
    view = wide[:, :K]
    if ops.gemm_skinny_supported(view, w):
        close(ops.gemm_skinny(view, w, b, out_dtype=torch.float32), view.double() @ w.double().t() + (b.double() if bias else 0), 1e-5)


def test_gemm_skinny_refuses_other_shapes():
    from ginfer_amd.kernels import ops, KernelError
    assert not ops.gemm_skinny_supported(rnd((65, 64), torch.bfloat16, 1), rnd((8, 64), torch.bfloat16, 2))
    assert not ops.gemm_skinny_supported(rnd((4, 12), torch.bfloat16, 1), rnd((8, 12), torch.bfloat16, 2))
    assert not ops.gemm_skinny_supported(rnd((4, 64), torch.float32, 1), rnd((8, 64), torch.float32, 2))
    with pytest.raises(KernelError):
        ops.gemm_skinny(rnd((65, 64), torch.bfloat16, 1), rnd((8, 64), torch.bfloat16, 2))


@pytest.mark.parametrize("M", [1, 5, 8, 33, 64])
@pytest.mark.parametrize("N,K", [(1536, 8960), (1536, 1536), (200, 4096), (777, 88)])
@pytest.mark.parametrize("nt,ks,gs", [(1, 8, 4), (2, 4, 2), (4, 8, 8), (1, 1, 3), (4, 2, 1), (2, 8, 1)])
@pytest.mark.parametrize("pack", [1, 2])
def test_gemm_skinny_tilings_and_split_parts(M, N, K, nt, ks, gs, pack):
    from ginfer_amd.kernels import ops
    if K // (gs * ks) < 8:
        pytest.skip("K too small for this split")
    if pack == 2 and M > 8:
        pytest.skip("packed tiles hold at most 8 rows")
    a, w, b = rnd((M, K), torch.bfloat16, 40), rnd((N, K), torch.bfloat16, 41), rnd((N,), torch.bfloat16, 42)
    ref = a.double() @ w.double().t() + b.double()
    out = ops.gemm_skinny(a, w, b, out_dtype=torch.float32, nt=nt, ks=ks, grid_splits=gs, pack=pack)
    if gs > 1:
        assert out.shape == (gs, M, N)
        # the norm that follows adds the parts to the residual stream
        res = rnd((M, N), torch.float32, 43)
        gain = torch.ones(N, dtype=torch.bfloat16, device=dev())
        r2 = res.clone()
        normed = ops.add_rmsnorm(r2, out, gain, 1e-6, torch.bfloat16)
        close(r2, res.double() + ref, 1e-5)
        close(normed, pm.rms_norm(res.double() + ref, gain.double(), 1e-6), 1e-2)
        out = out.sum(0)
    close(out, ref, 1e-5)


@pytest.mark.parametrize("M", [1, 5, 8, 16, 17, 64])
@pytest.mark.parametrize("I,K", [(8960, 1536), (160, 64), (136, 88), (448, 192),
                                 # from 2,048 columns on, up to 16 rows: the kernel that deals the columns evenly to a
                                 # multiple of 256 workgroups (one, two and three tiles a workgroup, uneven shares)
                                 (2056, 64), (6200, 40), (9000, 200), (12400, 24)])
def test_gemm_skinny_gated(M, I, K):
    from ginfer_amd.kernels import ops
    a, w = rnd((M, K), torch.bfloat16, 50), rnd((2 * I, K), torch.bfloat16, 51, scale=0.3)
    g, u = a.double() @ w[:I].double().t(), a.double() @ w[I:].double().t()
    ref = pm.swiglu(g, u)
    for pack in (1, 2) if M <= 8 else (1,):
        close(ops.gemm_skinny(a, w, gated=True, out_dtype=torch.float32, pack=pack), ref, 1e-5)
        close(ops.gemm_skinny(a, w, gated=True, pack=pack), ref, 1e-2)


@pytest.mark.parametrize("M", [1, 3, 8, 16])
@pytest.mark.parametrize("N,K,bias,gain_dtype", [(1536, 1536, False, torch.bfloat16), (1536, 8960, False, torch.float32),
                                                 (88, 136, True, torch.bfloat16), (200, 64, True, torch.float32),
                                                 (4096, 72, False, torch.bfloat16), (8192, 136, False, torch.bfloat16)])
def test_gemm_skinny_folds_the_norm_after_it(M, N, K, bias, gain_dtype):
    """The product that adds itself to the residual and hands on the norm's rows in two factors, and the
    products that take such rows: together they equal add, norm, product."""
    from ginfer_amd.kernels import ops
    eps = 1e-5
    a, w = rnd((M, K), torch.bfloat16, 70), rnd((N, K), torch.bfloat16, 71, scale=0.3)
    b = rnd((N,), torch.bfloat16, 72) if bias else None
    res0 = rnd((M, N), torch.float32, 73, scale=2.0)
    gain = (1 + 0.1 * rnd((N,), torch.float32, 74)).to(gain_dtype)
    assert ops.folded_norm_supported(a, w, res0, gain)
    res = res0.clone()
    rows = ops.gemm_skinny(a, w, b, into_norm=(res, gain, eps))
    h = res0.double() + a.double() @ w.double().t() + (b.double() if bias else 0)
    close(res, h, 1e-5)
    close(rows.scaled, h * gain.double(), 1e-2)
    close(rows.sumsq.sum(dim=1), (h * h).sum(dim=1), 1e-5)
    normed = pm.rms_norm(h, gain.double(), eps)
    close(rows.rows(), normed, 1e-2)
    # the partial sums come from the 32-bit residual that was written, column block by column block
    cols = -(-N // rows.sumsq.shape[1])             # a workgroup's columns: a tile's 16 or 8, or fewer (speed only)
    assert 1 <= cols <= 16 and rows.sumsq.shape[1] == -(-N // cols)
    parts = torch.stack([(res[:, c:c + cols].double() ** 2).sum(dim=1) for c in range(0, N, cols)], dim=1)
    close(rows.sumsq, parts, 1e-6)
    # products that take the rows: plain, gated, and the fused q|k|v projection
    w2 = rnd((72, N), torch.bfloat16, 75, scale=0.2)
    b2 = rnd((72,), torch.bfloat16, 76)
    given = rows.rows().double()          # what the rows stand for, from the rounded h * g
    close(ops.gemm_skinny(rows, w2, b2, out_dtype=torch.float32), given @ w2.double().t() + b2.double(), 1e-5)
    wg = rnd((2 * 40, N), torch.bfloat16, 77, scale=0.1)
    close(ops.gemm_skinny(rows, wg, gated=True, out_dtype=torch.float32),
          pm.swiglu(given @ wg[:40].double().t(), given @ wg[40:].double().t()), 1e-5)
    nh, nkv, hd = 3, 1, 32
    wq, bq = rnd(((nh + 2 * nkv) * hd, N), torch.bfloat16, 78, scale=0.1), rnd(((nh + 2 * nkv) * hd,), torch.bfloat16, 79)
    positions = torch.arange(M, dtype=torch.int32, device=dev()) * 7
    sin, cos = pm.rope_tables(1e4, hd, 200)
    kp, vp = rnd((4, nkv, 8, hd), torch.bfloat16, 80), rnd((4, nkv, hd, 8), torch.bfloat16, 81)
    slots = torch.arange(M, dtype=torch.int64, device=dev())
    q = ops.qkv_rope_skinny(rows, wq, bq, positions, cos.to(dev()), sin.to(dev()), slots, kp, vp, nh, nkv, hd)
    kp2, vp2 = kp.clone(), vp.clone()
    q2 = ops.qkv_rope_skinny(rows.rows().to(torch.bfloat16), wq, bq, positions, cos.to(dev()), sin.to(dev()), slots, kp2, vp2,
                             nh, nkv, hd)
    close(q, q2, 2e-2)
    close(kp, kp2, 2e-2)
    close(vp, vp2, 2e-2)
    # a row's factors do not depend on the rows beside it
    if M > 1:
        res1 = res0[M - 1:M].clone()
        alone = ops.gemm_skinny(a[M - 1:M], w, b, into_norm=(res1, gain, eps))
        if M <= 8:                                                       # the same tiling (packed tiles): bit for bit
            assert torch.equal(alone.scaled[0], rows.scaled[M - 1]) and torch.equal(alone.sumsq[0], rows.sumsq[M - 1])
            assert torch.equal(res1[0], res[M - 1])
        else:            # from 9 rows on the tiles are not packed: the same sums in another order
            close(res1[0], res[M - 1], 1e-6)
            close(alone.sumsq[0].sum(), rows.sumsq[M - 1].sum(), 1e-6)


def test_folded_norm_refuses_what_it_cannot_take():
    from ginfer_amd.kernels import ops, KernelError
    a, w = rnd((17, 64), torch.bfloat16, 1), rnd((32, 64), torch.bfloat16, 2)
    res, gain = rnd((17, 32), torch.float32, 3), rnd((32,), torch.bfloat16, 4)
    assert not ops.folded_norm_supported(a, w, res, gain)                       # more than 16 rows
    assert not ops.folded_norm_supported(a[:4], w, res[:4].bfloat16(), gain)    # residual not 32-bit
    assert not ops.folded_norm_supported(a[:4], w[:28], res[:4, :28], gain[:28])  # width no multiple of 8
    with pytest.raises(KernelError):
        ops.gemm_skinny(a, w, into_norm=(res, gain, 1e-6))


@pytest.mark.parametrize("M,parts", [(1, 1), (7, 3), (48, 4), (64, 2)])
@pytest.mark.parametrize("nh,nkv,hd,rd,theta,bias", [(12, 2, 128, 128, 1e4, True), (5, 1, 96, 96, 5e5, False), (4, 4, 64, 32, 1e4, True),
                                                     (3, 3, 48, 16, 1e6, True)])
@pytest.mark.parametrize("ps", [8, 12])
def test_rope_kv_from_parts(M, parts, nh, nkv, hd, rd, theta, bias, ps):
    """The rotation kernel on 32-bit partial sums of the projection: parts added in order, bias, rotation of q and k
    (a rotation of part of the head too), q out, k and v into their pages; nothing else touched."""
    from ginfer_amd.kernels import ops
    pages = 40
    width = (nh + 2 * nkv) * hd
    p = rnd((parts, M, width), torch.float32, 70)
    b = rnd((width,), torch.bfloat16, 71) if bias else None
    positions = torch.randint(0, 300, (M,), dtype=torch.int32, device=dev())
    sin, cos = pm.rope_tables(theta, rd, 300)
    slots = torch.randperm(pages * ps)[:M].to(torch.int64)
    if M > 1:
        slots[1] = -1
    kp, vp = rnd((pages, nkv, ps, hd), torch.bfloat16, 63), rnd((pages, nkv, hd, ps), torch.bfloat16, 64)
    kp0, vp0 = kp.clone().cpu(), vp.clone().cpu()
    q = ops.rope_kv_from_parts(p, b, positions, cos.to(dev()), sin.to(dev()), slots.to(dev()), kp, vp, nh, nkv, hd)
    assert q.dtype == torch.bfloat16 and q.shape == (M, nh * hd)
    y = p.double().cpu().sum(0) + (b.double().cpu() if bias else 0)
    pos = positions.cpu().tolist()
    qr = pm.apply_rope(y[:, :nh * hd].view(M, nh, hd), pos, sin.double(), cos.double()).reshape(M, -1)
    kr = pm.apply_rope(y[:, nh * hd:(nh + nkv) * hd].view(M, nkv, hd), pos, sin.double(), cos.double())
    v = y[:, (nh + nkv) * hd:].view(M, nkv, hd)
    close(q, qr, 1e-2)
    kpc, vpc = kp.float().cpu(), vp.float().cpu()
    touched_k, touched_v = torch.zeros_like(kpc, dtype=torch.bool), torch.zeros_like(vpc, dtype=torch.bool)
    for t in range(M):
        s = int(slots[t])
        if s < 0:
            continue
        close(kpc[s // ps, :, s % ps, :], kr[t], 1e-2)
        close(vpc[s // ps, :, :, s % ps], v[t], 1e-2)
        touched_k[s // ps, :, s % ps, :] = True
        touched_v[s // ps, :, :, s % ps] = True
    assert torch.equal(kp.cpu()[~touched_k], kp0[~touched_k]) and torch.equal(vp.cpu()[~touched_v], vp0[~touched_v])
    kp1, vp1 = kp0.clone().to(dev()), vp0.clone().to(dev())
    q2 = ops.rope_kv_from_parts(p, b, positions, cos.to(dev()), sin.to(dev()), slots.to(dev()), kp1, vp1, nh, nkv, hd,
                                write_kv=False)
    assert torch.equal(q2, q) and torch.equal(kp1.cpu(), kp0) and torch.equal(vp1.cpu(), vp0)


@pytest.mark.parametrize("M,pack", [(1, 1), (1, 2), (5, 2), (8, 1), (8, 2), (12, 1), (33, 1), (64, 1)])
@pytest.mark.parametrize("nh,nkv,hd,K,theta", [(12, 2, 128, 1536, 1e4), (6, 1, 32, 192, 1e6), (4, 4, 64, 88, 1e4), (5, 1, 96, 72, 5e5),
                                               (28, 4, 128, 72, 1e4)])     # the last: so many columns that tiles stay full
@pytest.mark.parametrize("ps", [8, 12])         # 12: the page of a slot by division, not by a shift
def test_qkv_rope_skinny(M, pack, nh, nkv, hd, K, theta, ps):
    """The fused decode kernel equals projection, then rotation and cache write."""
    from ginfer_amd.kernels import ops
    pages = 40
    width = (nh + 2 * nkv) * hd
    x, w, b = rnd((M, K), torch.bfloat16, 60), rnd((width, K), torch.bfloat16, 61, scale=0.2), rnd((width,), torch.bfloat16, 62)
    positions = torch.randint(0, 300, (M,), dtype=torch.int32, device=dev())
    sin, cos = pm.rope_tables(theta, hd, 300)
    slots = torch.randperm(pages * ps)[:M].to(torch.int64)
    if M > 1:
        slots[1] = -1
    kp, vp = rnd((pages, nkv, ps, hd), torch.bfloat16, 63), rnd((pages, nkv, hd, ps), torch.bfloat16, 64)
    kp0, vp0 = kp.clone().cpu(), vp.clone().cpu()
    assert ops.qkv_rope_skinny_supported(x, w, hd, hd)
    q = ops.qkv_rope_skinny(x, w, b, positions, cos.to(dev()), sin.to(dev()), slots.to(dev()), kp, vp, nh, nkv, hd,
                            pack=pack)
    y = x.double().cpu() @ w.double().cpu().t() + b.double().cpu()
    pos = positions.cpu().tolist()
    qr = pm.apply_rope(y[:, :nh * hd].view(M, nh, hd), pos, sin.double(), cos.double()).reshape(M, -1)
    kr = pm.apply_rope(y[:, nh * hd:(nh + nkv) * hd].view(M, nkv, hd), pos, sin.double(), cos.double())
    v = y[:, (nh + nkv) * hd:].view(M, nkv, hd)
    close(q, qr, 1e-2)
    kpc, vpc = kp.float().cpu(), vp.float().cpu()
    touched_k, touched_v = torch.zeros_like(kpc, dtype=torch.bool), torch.zeros_like(vpc, dtype=torch.bool)
    for t in range(M):
        s = int(slots[t])
        if s < 0:
            continue
        close(kpc[s // ps, :, s % ps, :], kr[t], 1e-2)
        close(vpc[s // ps, :, :, s % ps], v[t], 1e-2)
        touched_k[s // ps, :, s % ps, :] = True
        touched_v[s // ps, :, :, s % ps] = True
    assert torch.equal(kp.cpu()[~touched_k], kp0[~touched_k]) and torch.equal(vp.cpu()[~touched_v], vp0[~touched_v])
    # a run that reads another layer's cache writes nothing
    kp1, vp1 = kp0.clone().to(dev()), vp0.clone().to(dev())
    q2 = ops.qkv_rope_skinny(x, w, b, positions, cos.to(dev()), sin.to(dev()), slots.to(dev()), kp1, vp1, nh, nkv, hd,
                             write_kv=False, pack=pack)
    assert torch.equal(q2, q) and torch.equal(kp1.cpu(), kp0) and torch.equal(vp1.cpu(), vp0)
