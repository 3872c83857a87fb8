"""Each HIP kernel alone against a plain 32-bit torch formula of the same operation, at sizes
other than the engine's tests use: head sizes in steps of 16, head counts and groups that are no
power of two, widths and vocabularies that are no multiple of any tile.

bfloat16 bounds: inputs are exact in both; the kernel accumulates in 32-bit and rounds its
result once, so the error is half a unit in the last place of the result, 2**-9 relative, plus
the 32-bit summation error; the checks allow 2**-8 of the row's scale."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def dev(t):
    return t.to("cuda")


def tol(dtype, f32=2e-6, bf16=2 ** -8):
    return f32 if dtype == torch.float32 else bf16


def close(got, want, rel, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    scale = max(float(want.abs().max()), 1e-6)
    err = float((got - want).abs().max()) / scale
    assert err <= rel, f"{what}: error {err:.3e} of the scale exceeds {rel:.1e}"


def randn(*shape, dtype, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_and_gather(dtype):
    from inferrs_amd import ops
    table = randn(133, 72, dtype=dtype)
    ids = torch.tensor([0, 132, 5, 5, 77], dtype=torch.int32)
    assert torch.equal(ops.embed_gather(dev(table), dev(ids)).cpu(), table[ids.long()])
    assert torch.equal(ops.gather_rows(dev(table), dev(ids)).cpu(), table[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cols", [1, 40, 1000, 4096, 5120])
@pytest.mark.parametrize("add_one", [False, True])
def test_rmsnorm(dtype, cols, add_one):
    from inferrs_amd import ops
    x = randn(7, cols, dtype=dtype, seed=1, scale=3.0)
    d = randn(7, cols, dtype=dtype, seed=2)
    w = randn(cols, dtype=torch.float32, seed=3)
    eps = 1e-5

    def ref(v):
        v = v.float()
        return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * (w + 1.0 if add_one else w)
    close(ops.rmsnorm(dev(x), dev(w), eps, add_one), ref(x), tol(dtype), "rmsnorm")
    xs = dev(x.clone())
    out = ops.add_rmsnorm(xs, dev(d), dev(w), eps, add_one)
    summed = (x.float() + d.float()).to(dtype)
    assert torch.equal(xs.cpu(), summed), "add_rmsnorm must leave x + delta in x"
    close(out, ref(summed), tol(dtype), "add_rmsnorm")


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    from inferrs_amd import ops
    gu = randn(5, 2 * 203, dtype=dtype, seed=4, scale=4.0)
    g, u = gu[:, :203].float(), gu[:, 203:].float()
    close(ops.silu_mul(dev(gu)), g / (1 + torch.exp(-g)) * u, tol(dtype), "silu_mul")
    z = torch.zeros(1, 8, dtype=dtype)
    assert float(ops.silu_mul(dev(z)).abs().max()) == 0.0


def test_rope_table():
    from inferrs_amd import ops
    from inferrs_amd.parts.position import inverse_frequencies
    inv = torch.from_numpy(inverse_frequencies(1e6, 48))
    pos = torch.tensor([0, 1, 17, 4095, 40000], dtype=torch.int32)
    cos, sin = ops.rope_table(dev(pos), dev(inv))
    ang = (pos.float()[:, None] * inv[None, :]).double()          # the product itself is 32-bit
    assert float((cos.cpu().double() - torch.cos(ang)).abs().max()) < 2e-6
    assert float((sin.cpu().double() - torch.sin(ang)).abs().max()) < 2e-6
    assert inv[0].item() == 1.0


def ref_qk_rope(qkv, nq, nkv, d, qw, kw, eps, add_one, cos, sin, rot, interleaved):
    n = qkv.shape[0]
    x = qkv.float().view(n, nq + 2 * nkv, d)
    q, k, v = x[:, :nq], x[:, nq:nq + nkv], x[:, nq + nkv:]

    def norm(t, w):
        if w is None:
            return t
        return t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * (w + 1.0 if add_one else w)

    def rope(t):
        if cos is None:
            return t
        c, s = cos[:, None, :], sin[:, None, :]
        out = t.clone()
        if interleaved:
            a, b = t[..., 0:rot:2], t[..., 1:rot:2]
            out[..., 0:rot:2], out[..., 1:rot:2] = a * c - b * s, a * s + b * c
        else:
            a, b = t[..., :rot // 2], t[..., rot // 2:rot]
            out[..., :rot // 2], out[..., rot // 2:rot] = a * c - b * s, a * s + b * c
        return out
    return rope(norm(q, qw)), rope(norm(k, kw)), v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,rot,interleaved,normed", [
    (4, 2, 16, 16, False, True), (5, 1, 48, 48, False, True), (32, 8, 128, 128, False, True),
    (6, 3, 80, 32, False, False), (3, 3, 256, 64, True, True), (2, 1, 512, 512, False, True),
    (7, 7, 112, 0, False, True)])
def test_qk_rope_kv(dtype, nq, nkv, d, rot, interleaved, normed):
    from inferrs_amd import ops
    n, page, pages = 13, 4, 9
    qkv = randn(n, (nq + 2 * nkv) * d, dtype=dtype, seed=5, scale=2.0)
    qw = randn(d, dtype=torch.float32, seed=6) if normed else None
    kw = randn(d, dtype=torch.float32, seed=7) if normed else None
    g = torch.Generator().manual_seed(8)
    cos = torch.rand(n, rot // 2, generator=g) if rot else None
    sin = torch.rand(n, rot // 2, generator=g) if rot else None
    slots = torch.randperm(pages * page, generator=g)[:n].to(torch.int32)
    kc = torch.full((pages, nkv, page, d), 7.0, dtype=dtype)
    vc = torch.full((pages, nkv, d, page), 7.0, dtype=dtype)       # values: [dim][slot] inside a page
    kc_d, vc_d = dev(kc), dev(vc)
    q = ops.qk_rope_kv(dev(qkv), nq, nkv, d, q_norm_w=None if qw is None else dev(qw),
                       k_norm_w=None if kw is None else dev(kw), eps=1e-5, add_one=False,
                       cos=None if cos is None else dev(cos), sin=None if sin is None else dev(sin),
                       rot=rot, interleaved=interleaved, k_cache=kc_d, v_cache=vc_d, slots=dev(slots),
                       page_size=page)
    rq, rk, rv = ref_qk_rope(qkv, nq, nkv, d, qw, kw, 1e-5, False, cos, sin, rot, interleaved)
    close(q, rq, tol(dtype, 3e-6), "q")
    want_k, want_v = kc.float().clone(), vc.float().clone()
    for t in range(n):
        s = int(slots[t])
        want_k[s // page, :, s % page] = rk[t]
        want_v[s // page, :, :, s % page] = rv[t]
    close(kc_d, want_k, tol(dtype, 3e-6), "k cache")         # untouched slots keep their 7.0
    assert torch.equal(vc_d.cpu().float(), want_v.to(dtype).float()), "values are copied as they are"


@pytest.mark.parametrize("nq,nkv,d,page", [(8, 2, 128, 16), (3, 3, 64, 8), (2, 1, 256, 16), (5, 5, 48, 24),
                                            (4, 4, 128, 4)])
@pytest.mark.parametrize("layout", ["aligned", "shifted", "two requests", "shuffled"])
def test_qk_rope_kv_values_of_a_prompt_portion(nq, nkv, d, page, layout):
    """Steps with prompt portions write the values eight tokens at a time where their slots are
    neighbours in a page; every arrangement of the slots must end in the same cache."""
    from inferrs_amd import ops
    dtype, n, pages = torch.bfloat16, 43, 24
    g = torch.Generator().manual_seed(21)
    if layout == "aligned":
        slots = torch.arange(n) + 2 * page
    elif layout == "shifted":
        slots = torch.arange(n) + page + 3
    elif layout == "two requests":        # 19 tokens of one request, 24 of another, pages apart
        first_free = (page + 24 + page - 1) // page * page
        slots = torch.cat([torch.arange(19) + first_free + page + 5, torch.arange(24) + page])
    else:
        slots = torch.randperm(pages * page, generator=g)[:n]
    slots = slots.to(torch.int32)
    assert int(slots.max()) < pages * page and len(set(slots.tolist())) == n
    qkv = randn(n, (nq + 2 * nkv) * d, dtype=dtype, seed=22, scale=2.0)
    qw, kw = randn(d, dtype=torch.float32, seed=23), randn(d, dtype=torch.float32, seed=24)
    cos, sin = torch.rand(n, d // 2, generator=g), torch.rand(n, d // 2, generator=g)
    kc = torch.full((pages, nkv, page, d), 7.0, dtype=dtype)
    vc = torch.full((pages, nkv, d, page), 7.0, dtype=dtype)
    kc_d, vc_d = dev(kc), dev(vc)
    q = ops.qk_rope_kv(dev(qkv), nq, nkv, d, q_norm_w=dev(qw), k_norm_w=dev(kw), eps=1e-6, add_one=False,
                       cos=dev(cos), sin=dev(sin), rot=d, interleaved=False, k_cache=kc_d, v_cache=vc_d,
                       slots=dev(slots), page_size=page)
    rq, rk, rv = ref_qk_rope(qkv, nq, nkv, d, qw, kw, 1e-6, False, cos, sin, d, False)
    close(q, rq, tol(dtype, 3e-6), "q")
    want_k, want_v = kc.float().clone(), vc.float().clone()
    for t in range(n):
        s = int(slots[t])
        want_k[s // page, :, s % page] = rk[t]
        want_v[s // page, :, :, s % page] = rv[t]
    close(kc_d, want_k, tol(dtype, 3e-6), "k cache")
    assert torch.equal(vc_d.cpu().float(), want_v.to(dtype).float()), "values are copied as they are"
    # the kernel that decode steps use (a thread a head, values token by token) gives the same bits
    kc_1, vc_1 = dev(kc), dev(vc)
    ops.library().ia_qk_rope_kv_tune(0, 0)
    try:
        q_1 = ops.qk_rope_kv(dev(qkv), nq, nkv, d, q_norm_w=dev(qw), k_norm_w=dev(kw), eps=1e-6, add_one=False,
                             cos=dev(cos), sin=dev(sin), rot=d, interleaved=False, k_cache=kc_1, v_cache=vc_1,
                             slots=dev(slots), page_size=page)
    finally:
        ops.library().ia_qk_rope_kv_tune(1, 1)
    assert torch.equal(q, q_1) and torch.equal(kc_d, kc_1) and torch.equal(vc_d, vc_1)


def ref_attention(q, kc, vc, positions, token_seq, table, window, scale):
    n, nq, d = q.shape
    nkv, page = kc.shape[1], kc.shape[2]
    out = torch.zeros(n, nq, d)
    for t in range(n):
        pos = int(positions[t])
        lo = max(0, pos - window + 1) if window else 0
        keys = list(range(lo, pos + 1))
        pg = [int(table[int(token_seq[t]), j // page]) for j in keys]
        for h in range(nq):
            kvh = h // (nq // nkv)
            k = torch.stack([kc[p, kvh, j % page] for p, j in zip(pg, keys)]).float()
            v = torch.stack([vc[p, kvh, :, j % page] for p, j in zip(pg, keys)]).float()
            s = (k @ q[t, h].float()) * scale
            out[t, h] = torch.softmax(s, 0) @ v
    return out


def ref_attention_dense(q, kc, vc, positions, token_seq, table, window, scale):
    """The same formula, request by request on dense copies of its keys and values (for long cases)."""
    n, nq, d = q.shape
    nkv, page = kc.shape[1], kc.shape[2]
    out = torch.zeros(n, nq, d)
    for s in token_seq.unique().tolist():
        rows = (token_seq == s).nonzero().flatten()
        pos = positions[rows].long()
        length = int(pos.max()) + 1
        pages = table[s, :-(-length // page)].long()
        k = kc[pages].float().permute(1, 0, 2, 3).reshape(nkv, -1, d)[:, :length]           # [nkv, L, d]
        v = vc[pages].float().permute(1, 0, 3, 2).reshape(nkv, -1, d)[:, :length]           # [nkv, L, d]
        k, v = k.repeat_interleave(nq // nkv, 0), v.repeat_interleave(nq // nkv, 0)         # [nq, L, d]
        sc = torch.einsum("thd,hjd->thj", q[rows].float(), k) * scale
        j = torch.arange(length)
        hidden = j[None, :] > pos[:, None]
        if window:
            hidden |= j[None, :] < (pos[:, None] - window + 1)
        sc = sc.masked_fill(hidden[:, None, :], float("-inf"))
        out[rows] = torch.einsum("thj,hjd->thd", torch.softmax(sc, -1), v)
    return out


def attention_case(dtype, nq, nkv, d, page, lens, q_lens, seed, needle=False):
    """Requests with `lens` cached tokens of which the last `q_lens` are this step's queries,
    pages handed out in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    n_seqs = len(lens)
    max_pages = max(-(-l // page) for l in lens)
    total_pages = sum(-(-l // page) for l in lens) + 3
    perm = torch.randperm(total_pages, generator=g).tolist()
    table = torch.zeros(n_seqs, max_pages, dtype=torch.int32)
    for s, l in enumerate(lens):
        for j in range(-(-l // page)):
            table[s, j] = perm.pop()
    kc = randn(total_pages, nkv, page, d, dtype=dtype, seed=seed + 1)
    vc = randn(total_pages, nkv, d, page, dtype=dtype, seed=seed + 2)
    positions = torch.tensor([p for l, ql in zip(lens, q_lens) for p in range(l - ql, l)], dtype=torch.int32)
    token_seq = torch.tensor([s for s, ql in enumerate(q_lens) for _ in range(ql)], dtype=torch.int32)
    q = randn(len(positions), nq, d, dtype=dtype, seed=seed + 3)
    if needle:
        # one far key per request that every query of head 0 points at: its score stands out,
        # so the output is that key's value unless the key is lost
        for s, l in enumerate(lens):
            j = l // 3
            kc[int(table[s, j // page]), 0, j % page] = (q[token_seq == s][-1, 0].float() * 4).to(dtype)
    return q, kc, vc, positions, token_seq, table


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,page,window", [
    (4, 2, 16, 4, None), (5, 1, 48, 16, None), (8, 1, 128, 16, None), (6, 3, 32, 8, 37),
    (3, 3, 80, 5, None), (2, 2, 256, 16, 100)])
def test_attention_generic(dtype, nq, nkv, d, page, window):
    from inferrs_amd import ops
    lens, q_lens = [1, 70, 129, 200, 64], [1, 70, 2, 1, 17]
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, page, lens, q_lens, 11, needle=True)
    scale = 1.0 / math.sqrt(d)
    got = ops.attention_generic(dev(q), dev(kc), dev(vc), dev(positions), dev(token_seq), dev(table),
                                window=window, scale=scale)
    want = ref_attention(q, kc, vc, positions, token_seq, table, window, scale)
    close(got, want, tol(dtype, 5e-6, 2 ** -7), "attention")
    close(ref_attention_dense(q, kc, vc, positions, token_seq, table, window, scale), want, 1e-5, "the two references")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,page,window", [
    (8, 2, 128, 16, None), (3, 1, 72, 8, None), (5, 5, 24, 5, None), (10, 2, 64, 16, 700), (2, 1, 320, 32, None)])
def test_attention_generic_in_segments_is_the_same_bits_as_in_one_walk(dtype, nq, nkv, d, page, window):
    """Keys beyond one segment of 512: a wave a segment with the merge kernel behind it (steps of few tokens)
    against one wave that walks all segments of its token (steps of many tokens), bit for bit, and both against
    the reference; head sizes and page sizes that are no multiple of four take the loads of single elements.
    What the pages hold beyond a request's keys is NaN."""
    from inferrs_amd import ops
    lens, q_lens = [1500, 513, 1024, 40], [2, 1, 3, 1]
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, page, lens, q_lens, 29, needle=True)
    want = ref_attention_dense(q, kc, vc, positions, token_seq, table, window, 1.0 / math.sqrt(d))
    for s, l in enumerate(lens):                     # the rest of every request's last page
        if l % page:
            kc[int(table[s, l // page]), :, l % page:] = float("nan")
            vc[int(table[s, l // page]), :, :, l % page:] = float("nan")
    args = (dev(q), dev(kc), dev(vc), dev(positions), dev(token_seq), dev(table))
    scale = 1.0 / math.sqrt(d)
    whole = ops.attention_generic(*args, window=window, scale=scale, split=False)
    parts = ops.attention_generic(*args, window=window, scale=scale, split=True)
    bound = ops.attention_generic(*args, window=window, scale=scale, split=True, max_kv_len=max(lens))
    assert torch.equal(whole, parts) and torch.equal(whole, bound)
    close(whole, want, tol(dtype, 5e-6, 2 ** -7), "attention in segments")
    assert ops.library().ia_attention_generic_workspace(4096, nq, nkv, d, 2000) == 0          # tokens enough: no split
    with pytest.raises(ops.KernelError):
        ops.attention_generic(*args, window=window, scale=scale, split=True, max_kv_len=300)  # one segment: nothing to split


@pytest.mark.parametrize("nq,nkv,d,page,window", [
    (4, 2, 16, 16, None), (5, 1, 48, 16, None), (8, 1, 128, 16, None), (32, 8, 128, 16, None),
    (6, 3, 32, 32, 37), (3, 3, 80, 16, None), (2, 2, 256, 64, 100), (40, 2, 64, 16, None), (7, 7, 112, 48, 5)])
@pytest.mark.parametrize("lens,q_lens", [
    ([1, 70, 129, 200, 64], [1, 70, 2, 1, 17]),          # mixed: whole prompts, portions, single tokens
    ([300, 17, 1000, 33], [1, 1, 1, 1]),                  # decode only
    ([257], [257]), ([16], [16]), ([32, 31, 33], [3, 31, 1])])
def test_attention_mfma(nq, nkv, d, page, window, lens, q_lens):
    from inferrs_amd import ops
    dtype = torch.bfloat16
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, page, lens, q_lens, 13, needle=True)
    # slots past a request's length hold NaN: they must not reach the result
    for s, l in enumerate(lens):
        for j in range(l, -(-l // page) * page):
            kc[int(table[s, j // page]), :, j % page] = float("nan")
            vc[int(table[s, j // page]), :, :, j % page] = float("nan")
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    want = ref_attention(q, kc, vc, positions, token_seq, table, window, scale)
    for splits in (None, 1, 2, 8):
        got = ops.attention_mfma(dev(q), dev(kc), dev(vc), dev(positions), dev(cu), dev(table),
                                 max_q_len=max(q_lens), max_kv_len=max(lens), window=window, scale=scale,
                                 splits=splits)
        close(got, want, 2 ** -7, f"attention_mfma splits={splits}")


@pytest.mark.parametrize("nq,nkv,page,window", [(8, 2, 16, None), (4, 4, 32, None), (10, 2, 48, None), (8, 2, 16, 150),
                                                (32, 8, 16, None)])
@pytest.mark.parametrize("lens,q_lens", [
    ([333], [333]),                                       # a whole prompt
    ([700, 90], [130, 64]),                               # late portions of long prompts
    ([64, 65, 127, 128], [64, 65, 127, 128]),             # around the size of a stage of keys
    ([500, 40, 260], [37, 40, 1])])                       # short portions and a single token beside a long one
def test_attention_mfma_prompt_portions_head_size_128(nq, nkv, page, window, lens, q_lens):
    """Head size 128 with 128 columns or more: blocks of four waves that share keys and values through
    shared memory, against the reference and against the kernel of single waves."""
    from inferrs_amd import ops
    dtype, d = torch.bfloat16, 128
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, page, lens, q_lens, 17, needle=True)
    for s, l in enumerate(lens):
        for j in range(l, -(-l // page) * page):
            kc[int(table[s, j // page]), :, j % page] = float("nan")
            vc[int(table[s, j // page]), :, :, j % page] = float("nan")
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    want = ref_attention_dense(q, kc, vc, positions, token_seq, table, window, scale)
    args = (dev(q), dev(kc), dev(vc), dev(positions), dev(cu), dev(table))
    kw = dict(max_q_len=max(q_lens), max_kv_len=max(lens), window=window, scale=scale, splits=1)
    got = ops.attention_mfma(*args, **kw)
    close(got, want, 2 ** -7, "blocks of four waves")
    for splits in (None, 2, 3):                        # the keys shared out between blocks and merged
        close(ops.attention_mfma(*args, **dict(kw, splits=splits)), want, 2 ** -7, f"blocks of four waves, splits={splits}")
    lib = ops.library("attn_d128")
    lib.ia_attention_mfma_tiles(0)
    try:
        single = ops.attention_mfma(*args, **kw)
    finally:
        lib.ia_attention_mfma_tiles(1)
    close(single, want, 2 ** -7, "single waves")
    close(got, single.float().cpu(), 2 ** -7, "the two kernels")
    # blocks of 64 columns and of 128 (the launch picks by the step's size; here each is forced): a column's keys are
    # walked in the same order with the same arithmetic, so the bits are the same, with the keys split as well.  (Under a
    # window a block's walk begins at the first stage that any of its columns sees, and which of the block's two
    # groups of waves takes a stage follows from there: another width of block, another pairing, the same sums in
    # another order.)
    for splits in (1, 2, 3):
        outs = []
        for columns in (2, 3):
            lib.ia_attention_mfma_tiles(columns)
            try:
                outs.append(ops.attention_mfma(*args, **dict(kw, splits=splits)))
            finally:
                lib.ia_attention_mfma_tiles(1)
        if window is None:
            assert torch.equal(outs[0], outs[1]), f"blocks of 64 and of 128 columns, splits={splits}"
        close(outs[1], want, 2 ** -7, f"blocks of 128 columns, splits={splits}")
        close(outs[0], want, 2 ** -7, f"blocks of 64 columns, splits={splits}")


def test_attention_mfma_prompt_that_half_fills_the_chip():
    """Between one and two blocks a compute unit the second half of the blocks walks its tiles in the other
    order; with 47 tiles a row of the grid that half does not begin at a row's start."""
    from inferrs_amd import ops
    dtype, d, nq, nkv, page = torch.bfloat16, 128, 32, 8, 16
    lens = q_lens = [1500]
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, page, lens, q_lens, 19, needle=True)
    cu = torch.tensor([0, 1500], dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    want = ref_attention_dense(q, kc, vc, positions, token_seq, table, None, scale)
    got = ops.attention_mfma(dev(q), dev(kc), dev(vc), dev(positions), dev(cu), dev(table), max_q_len=1500,
                             max_kv_len=1500, window=None, scale=scale, splits=1)
    close(got, want, 2 ** -7, "47 x 8 blocks")


def test_attention_mfma_refuses_what_it_cannot_take():
    from inferrs_amd import ops
    q, kc, vc, positions, token_seq, table = attention_case(torch.bfloat16, 2, 1, 16, 8, [9], [9], 1)
    cu = torch.tensor([0, 9], dtype=torch.int32)
    with pytest.raises(ops.KernelError, match="page sizes in steps of 16"):
        ops.attention_mfma(dev(q), dev(kc), dev(vc), dev(positions), dev(cu), dev(table), max_q_len=9,
                           max_kv_len=9, window=None, scale=0.25)


def test_gemm_reference_products():
    # candle-core/tests/matmul_tests.rs:18-33 and candle-nn/src/linear.rs:7-20
    from inferrs_amd import ops
    a = torch.tensor([[1., 2.], [3., 4.]])
    b = torch.tensor([[4., 5.], [6., 7.]])
    assert ops.linear(dev(a), dev(b.t().contiguous())).cpu().tolist() == [[16., 19.], [36., 43.]]
    w = torch.tensor([[1., 2.], [3., 4.], [5., 6.]])
    assert ops.linear(dev(torch.tensor([[10., 100.]])), dev(w)).cpu().tolist() == [[210., 430., 650.]]


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 130, 40), (65, 64, 64), (17, 515, 136), (130, 72, 200), (2, 7, 1000),
                                   (200, 300, 136), (300, 1000, 520), (16, 100, 1000), (129, 128, 4), (140, 131, 42)])
def test_gemm_tiled_float32_is_true_32_bit(m, n, k):
    """Three kernels share this product: one for up to 16 rows, tiles of 64 x 64, and tiles of 128 x 128 for more than 128
    rows (k a multiple of 4); each adds an output up with k ascending, so they give the same bits."""
    from inferrs_amd import ops
    x, w = randn(m, k, dtype=torch.float32, seed=1), randn(n, k, dtype=torch.float32, seed=2)
    want = (x.double() @ w.double().t())
    whole = ops.linear(dev(x), dev(w)).cpu()
    # a reduced-precision matrix mode (tf32-like, 10 bits) would be off by about 1e-3
    assert float((whole.double() - want).abs().max()) <= 4e-6 * max(1.0, float(want.abs().max()))
    # rows do not depend on what else is in the batch: alone, among 16, among 40 and among all
    for rows in (1, 16, 40):
        rows = min(rows, m)
        assert torch.equal(ops.linear(dev(x[m - rows:]), dev(w)).cpu(), whole[m - rows:])


@pytest.mark.parametrize("m", [1, 2, 8, 12, 13, 16, 17, 33, 64, 65, 200])
# (5,120 features: blocks of 10; 5,120 wide: k shared out between 10 waves)
@pytest.mark.parametrize("n,k", [(130, 40), (515, 136), (4096, 4096), (1000, 12288), (16, 8), (5120, 5120), (7170, 5128)])
@pytest.mark.parametrize("out_dtype", DTYPES)
def test_linear_bfloat16(m, n, k, out_dtype):
    from inferrs_amd import ops
    x, w = randn(m, k, dtype=torch.bfloat16, seed=1), randn(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    want = x.double() @ w.double().t()
    got = ops.linear(dev(x), dev(w), out_dtype)
    assert got.dtype == out_dtype
    # beyond the skinny kernel's rows a 32-bit result is the vendor's bfloat16 one widened
    close(got, want, tol(out_dtype, 2e-5) if m <= ops.SKINNY_MAX_ROWS else 2 ** -8, f"linear {m}x{n}x{k}")


@pytest.mark.parametrize("dual", [False, True])
@pytest.mark.parametrize("m,n,k", [(1, 16, 64), (255, 250, 64), (256, 256, 128), (257, 260, 192), (777, 1002, 320),
                                   (2048, 1536, 4096), (300, 130, 1024)])
def test_tiled_matrix_core_product(m, n, k, dual):
    """The tiled kernel for many rows, alone: sizes that fill no tile, one and several stages of k, features that
    are no multiple of four (single stores), with and without the activation inside."""
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=1)
    w = randn((2 if dual else 1) * n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    got = ops.gemm_mfma_bf16(dev(x), dev(w), dual)
    assert got.shape == (m, n) and got.dtype == torch.bfloat16
    want = x.double() @ w.double().t()
    if dual:
        gate, up = want[:, :n].to(torch.bfloat16).double(), want[:, n:].to(torch.bfloat16).double()
        want = gate / (1 + torch.exp(-gate)) * up
    close(got, want, 2 ** -7, f"tiled {m}x{n}x{k} dual={dual}")


def test_tiled_matrix_core_product_refuses_other_widths():
    from inferrs_amd import ops
    with pytest.raises(ops.KernelError):
        ops.gemm_mfma_bf16(dev(randn(32, 40, dtype=torch.bfloat16)), dev(randn(16, 40, dtype=torch.bfloat16)))


@pytest.mark.parametrize("m", [1, 12])
@pytest.mark.parametrize("n,k", [(5120, 17408), (5120, 25600), (10240, 5120)])
def test_linear_bfloat16_long_rows(m, n, k):
    """Widths whose k steps do not divide evenly between the waves: the last wave takes what is left."""
    from inferrs_amd import ops
    x, w = randn(m, k, dtype=torch.bfloat16, seed=1), randn(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    close(ops.linear(dev(x), dev(w), torch.float32), x.double() @ w.double().t(), 2e-5, f"linear {m}x{n}x{k}")


@pytest.mark.parametrize("m", [1, 8, 17, 40, 64])
@pytest.mark.parametrize("n,k", [(130, 40), (12288, 4096), (200, 136), (17408, 5120)])
def test_gated_silu_linear(m, n, k):
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=1)
    w = randn(2 * n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    gate = (x.double() @ w[:n].double().t()).to(torch.bfloat16).double()     # the products are stored, then activated
    up = (x.double() @ w[n:].double().t()).to(torch.bfloat16).double()
    want = gate / (1 + torch.exp(-gate)) * up
    close(ops.gated_silu_linear(dev(x), dev(w)), want, 2 ** -7, "fused")
    close(ops.silu_mul(ops.linear(dev(x), dev(w))), want, 2 ** -7, "two kernels")


class _Norm:
    """What the products need of a norm part."""
    def __init__(self, weight, add_one=False):
        self.weight, self.add_one, self.eps = weight, add_one, 1e-6


@pytest.mark.parametrize("m", [1, 2, 8, 12, 13, 16])
@pytest.mark.parametrize("n,k,n2,add_one", [(4096, 4096, 6144, False), (4096, 12288, 6144, False), (2560, 1024, 520, True),
                                            (5120, 8192, 7168, False),
                                            (144, 4096, 4096, False), (200, 40, 72, False)])
def test_products_around_a_residual_stream(m, n, k, n2, add_one):
    """A product that adds itself to the stream (leaving the rows' sums of squares and the rows times the next
    norm's weight), and the product after it, which finishes the norm by scaling its sums: the stream holds
    the bits that the add kernel would leave, and the second product is the product of the normed rows up to
    where the one rounding of a normed value happens."""
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=31)
    w = randn(n, k, dtype=torch.bfloat16, seed=32, scale=0.03)
    stream = randn(m, n, dtype=torch.bfloat16, seed=33)
    norm_w = (0.0 if add_one else 1.0) + 0.1 * randn(n, dtype=torch.float32, seed=34)
    w2 = randn(n2, n, dtype=torch.bfloat16, seed=35, scale=0.03)
    w3 = randn(2 * n2, n, dtype=torch.bfloat16, seed=36, scale=0.03)
    # the two-kernel way
    plain_stream = dev(stream)
    plain_rows = ops.add_rmsnorm(plain_stream, ops.gemm_skinny_bf16(dev(x), dev(w)), dev(norm_w), 1e-6, add_one)
    # the products' way
    fused_stream = dev(stream)
    norm = _Norm(dev(norm_w), add_one)
    sums, scaled = ops.linear_add(dev(x), dev(w), fused_stream, norm)
    per = ops.library().ia_gemm_skinny_block_rows(n)              # features a block: 16, fewer where that fills the chip evenly
    assert 8 <= per <= 16 and tuple(sums.shape) == (m, -(-n // per)) and scaled.shape == fused_stream.shape
    assert torch.equal(fused_stream, plain_stream), "the stream after the sum"
    new_rows = fused_stream.float().cpu().double()
    want_sums = torch.nn.functional.pad(new_rows.pow(2), (0, -n % per)).view(m, -1, per).sum(-1)
    close(sums, want_sums, 1e-5, "sums of squares")
    gain = norm_w.double() + (1.0 if add_one else 0.0)
    assert torch.equal(scaled.cpu(), (new_rows * gain).to(torch.float32).to(torch.bfloat16)), "rows times the weight"
    rows = ops.NormedRows(fused_stream, scaled, sums, norm.weight, 1e-6, add_one)
    assert torch.equal(rows.materialize(), plain_rows)
    exact = new_rows / torch.sqrt(new_rows.pow(2).mean(-1, keepdim=True) + 1e-6) * gain
    g = (exact @ w3[:n2].double().t()).to(torch.bfloat16).double()
    refs = {"product": exact @ w2.double().t(),
            "gated product": g / (1 + torch.exp(-g)) * (exact @ w3[n2:].double().t()).to(torch.bfloat16).double()}
    for what, got, want in (("product", ops.linear(rows, dev(w2)), ops.linear(plain_rows, dev(w2))),
                            ("gated product", ops.gated_silu_linear(rows, dev(w3)), ops.gated_silu_linear(plain_rows, dev(w3)))):
        close(want, refs[what], 2 ** -6, what + " of the two kernels")
        close(got, refs[what], 2 ** -6, what + " with the norm's end inside")
    # without a next norm: sums only
    only = ops.linear_add(dev(x), dev(w), dev(stream))
    assert only[1] is None and torch.equal(only[0], sums)


@pytest.mark.parametrize("m", [1, 8, 16])
@pytest.mark.parametrize("blocks", [32, 30])
def test_gated_product_of_few_normed_rows_on_blocks_that_fill_the_chip(m, blocks, monkeypatch):
    """A [gate; up] whose blocks fill the chip evenly (12,288 features: 256 blocks of 48) takes the kernel of 17 to 64
    rows also for few rows, with the norm's end inside (the rows' sums of squares, in fours or one by one): against the
    exact result, against the skinny product's way, and a row does not depend on its batch."""
    from inferrs_amd import ops
    k, n2 = 512, 12288
    x = randn(m, k, dtype=torch.bfloat16, seed=41, scale=2.0)
    gain = 1.0 + 0.1 * randn(k, dtype=torch.float32, seed=42)
    w3 = dev(randn(2 * n2, k, dtype=torch.bfloat16, seed=43, scale=0.05))
    scaled = (x.float() * gain).to(torch.bfloat16)
    sums = x.float().pow(2).view(m, blocks, -1).sum(-1) if k % blocks == 0 else \
        torch.cat([x.float().pow(2)[:, :17 * (blocks - 1)].reshape(m, blocks - 1, 17).sum(-1),
                   x.float().pow(2)[:, 17 * (blocks - 1):].sum(-1, keepdim=True)], 1)
    assert sums.shape == (m, blocks)
    rows = ops.NormedRows(dev(x), dev(scaled), dev(sums.contiguous()), dev(gain), 1e-6, False)
    assert ops.library().ia_gemm_mid_fills(n2, k, 1) == 1
    with ops.KernelTimer() as timer:
        got = ops.gated_silu_linear(rows, w3)
    assert set(timer.summary()) == {"gemm_mid_bf16_scaled"}
    part = ops.NormedRows(dev(x[m // 3:]), dev(scaled[m // 3:].contiguous()), dev(sums[m // 3:].contiguous()), dev(gain), 1e-6, False)
    assert torch.equal(ops.gated_silu_linear(part, w3), got[m // 3:])
    monkeypatch.setattr(ops, "MID_PRODUCTS", "library")
    with ops.KernelTimer() as timer:
        skinny = ops.gated_silu_linear(rows, w3)
    assert set(timer.summary()) == {"gemm_skinny_stream"}
    exact = scaled.double() / torch.sqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-6)
    g = (exact @ w3[:n2].double().cpu().t()).to(torch.bfloat16).double()
    want = g / (1 + torch.exp(-g)) * (exact @ w3[n2:].double().cpu().t()).to(torch.bfloat16).double()
    close(got, want, 2 ** -6, "with the norm's end inside")
    close(got, skinny, 2 ** -7, "against the skinny product")


def test_products_leave_the_stream_alone_where_they_cannot_take_it():
    from inferrs_amd import ops
    # more rows than the skinny product takes, or a 32-bit stream: the product does not add itself
    many = ops.SKINNY_MAX_ROWS + 1
    big = randn(many, 64, dtype=torch.bfloat16, seed=3)
    assert ops.linear_add(dev(big), dev(randn(64, 64, dtype=torch.bfloat16, seed=4)), dev(randn(many, 64, dtype=torch.bfloat16, seed=5))) is None
    x, w = randn(3, 40, dtype=torch.float32, seed=1), randn(64, 40, dtype=torch.float32, seed=2)
    assert ops.linear_add(dev(x), dev(w), dev(torch.zeros(3, 64))) is None
    # a product of 65536 features and more (a logits head) norms the rows first
    xs = randn(2, 64, dtype=torch.bfloat16, seed=6)
    rows = ops.NormedRows(dev(xs), dev(xs), dev((xs.float() ** 2).sum(-1, keepdim=True)), dev(torch.ones(64)), 1e-6, False)
    head = dev(randn(65536, 64, dtype=torch.bfloat16, seed=7))
    assert torch.equal(ops.linear(rows, head), ops.linear(ops.rmsnorm(dev(xs), dev(torch.ones(64)), 1e-6, False), head))


def test_skinny_rows_do_not_depend_on_the_batch():
    from inferrs_amd import ops
    x, w = randn(16, 4096, dtype=torch.bfloat16, seed=1), randn(77, 4096, dtype=torch.bfloat16, seed=2)
    full = ops.gemm_skinny_bf16(dev(x), dev(w), torch.float32).cpu()
    assert torch.equal(ops.gemm_skinny_bf16(dev(x[:1]), dev(w), torch.float32).cpu(), full[:1])
    assert torch.equal(ops.gemm_skinny_bf16(dev(x[3:9].contiguous()), dev(w), torch.float32).cpu(), full[3:9])


def _without_staging(fn):
    """The skinny product's plain variant: the tuning entry switches the staged ones off (and on again)."""
    from inferrs_amd import ops
    lib = ops.library()
    lib.ia_gemm_skinny_tune(2048, 8, 5, 8, 0)
    try:
        return fn()
    finally:
        lib.ia_gemm_skinny_tune(2048, 8, 5, 8, 1)


def test_skinny_variants_for_one_round_weights_agree_bit_for_bit():
    # a weight of fewer than three blocks a compute unit whose waves take whole chunks of 16 k steps: its
    # activations are staged through shared memory; the plain variant gives the same bits
    from inferrs_amd import ops
    n, k = 4096, 4096
    x = randn(16, k, dtype=torch.bfloat16, seed=1)
    w = randn(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    full = ops.gemm_skinny_bf16(dev(x), dev(w), torch.float32).cpu()
    close(full, x.double() @ w.double().t(), 2e-5, "one round")
    assert torch.equal(_without_staging(lambda: ops.gemm_skinny_bf16(dev(x), dev(w), torch.float32).cpu()), full)
    for lo, hi in ((0, 1), (7, 8), (3, 9), (0, 12), (2, 15)):
        part = ops.gemm_skinny_bf16(dev(x[lo:hi].contiguous()), dev(w), torch.float32).cpu()
        assert torch.equal(part, full[lo:hi]), (lo, hi)
        assert torch.equal(_without_staging(lambda: ops.gemm_skinny_bf16(dev(x[lo:hi].contiguous()), dev(w), torch.float32).cpu()),
                           part), (lo, hi)


@pytest.mark.parametrize("dual", [False, True])
def test_skinny_variants_for_tall_weights_agree_bit_for_bit(dual):
    # a weight with three blocks a compute unit and more takes the variant that stages the activations through
    # shared memory while two blocks fit a compute unit, the plain one beyond; both give the same bits
    from inferrs_amd import ops
    n, k = 8200, 520
    x = randn(16, k, dtype=torch.bfloat16, seed=1)
    w = randn(2 * n if dual else n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    full = ops.gemm_skinny_bf16(dev(x), dev(w), torch.float32, dual=dual).cpu()
    if dual:
        gate = (x.double() @ w[:n].double().t()).to(torch.bfloat16).double()
        want = gate / (1 + torch.exp(-gate)) * (x.double() @ w[n:].double().t()).to(torch.bfloat16).double()
        close(full, want, 2 ** -7, "dual")
    else:
        close(full, x.double() @ w.double().t(), 2e-5, "tall")
    assert torch.equal(_without_staging(lambda: ops.gemm_skinny_bf16(dev(x), dev(w), torch.float32, dual=dual).cpu()), full)
    for lo, hi in ((0, 1), (3, 9), (0, 12), (5, 7), (2, 15)):
        part = ops.gemm_skinny_bf16(dev(x[lo:hi].contiguous()), dev(w), torch.float32, dual=dual).cpu()
        assert torch.equal(part, full[lo:hi]), (lo, hi)


def test_argmax_lowest_index_among_equal_maxima():
    from inferrs_amd import ops
    z = randn(4, 151936, dtype=torch.float32, seed=3)
    z[1, 150000] = z[1, 77] = 9.0
    z[2, :] = 0.0
    z[3, 151935] = 10.0
    got = ops.argmax(dev(z)).cpu().tolist()
    assert got == [int(torch.argmax(z[0])), 77, 0, 151935]
    small = torch.tensor([[1.0, 3.0, 3.0]])
    assert ops.argmax(dev(small)).cpu().tolist() == [1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_fill_normal_equals_the_host_fill(dtype):
    from inferrs_amd import ops
    from inferrs_amd.weights.random_init import normal_values
    n, seed = 300_001, 0x1234_5678_9ABC_DEF0
    host = torch.from_numpy(normal_values(n, seed, 1.0, 0.1)).to(dtype)
    got = ops.fill_normal((n,), seed, 1.0, 0.1, dtype, "cuda").cpu()
    # the two differ only where the device's and NumPy's 64-bit log or cosine differ in their last
    # bit AND that falls on a rounding boundary of the narrower type: (almost) never
    assert int((got != host).sum()) <= (3 if dtype == torch.float32 else 0)
    z = (ops.fill_normal((n,), 7, 0.0, 1.0, torch.float32, "cuda").cpu()).double()
    assert abs(float(z.mean())) < 0.01 and abs(float(z.std()) - 1.0) < 0.01
    assert abs(float((z ** 4).mean()) - 3.0) < 0.1                      # the fourth moment of a normal


@pytest.mark.parametrize("nq,nkv,d,page,window", [
    (32, 8, 128, 16, None), (4, 2, 64, 16, None), (40, 2, 64, 32, None), (6, 3, 192, 16, 37), (2, 1, 256, 48, None)])
@pytest.mark.parametrize("norm,rope,write", [(True, True, True), (False, True, True), (True, False, True), (True, True, False)])
def test_attention_decode_fused_is_the_three_kernels_in_one(nq, nkv, d, page, window, norm, rope, write):
    """Decode steps: per-head norm, rotation, cache write and attention in one kernel against the separate
    kernels (the same arithmetic but for the order of the norm's sum of squares): the results agree to
    the rounding of bfloat16, and the cache holds the same new keys and values."""
    from inferrs_amd import ops
    dtype = torch.bfloat16
    lens = [300, 17, 1000, 33, 64, 1]                       # lengths after the step; the last token of each is this step's
    q, kc, vc, positions, token_seq, table = attention_case(dtype, nq, nkv, d, page, lens, [1] * len(lens), 23)
    n = len(lens)
    qkv = randn(n, (nq + 2 * nkv) * d, dtype=dtype, seed=5)
    qw = (1 + 0.3 * randn(d, dtype=torch.float32, seed=6)) if norm else None
    kw = (1 + 0.3 * randn(d, dtype=torch.float32, seed=7)) if norm else None
    cos = sin = None
    if rope:
        inv = 1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        ang = positions.float()[:, None] * inv[None, :]
        cos, sin = torch.cos(ang), torch.sin(ang)
    slots = torch.tensor([int(table[s, (l - 1) // page]) * page + (l - 1) % page for s, l in enumerate(lens)], dtype=torch.int32)
    cu = torch.arange(n + 1, dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    dv = lambda t: None if t is None else dev(t)
    # the separate kernels
    k1, v1 = dev(kc), dev(vc)
    q1 = ops.qk_rope_kv(dev(qkv), nq, nkv, d, q_norm_w=dv(qw), k_norm_w=dv(kw), eps=1e-5, add_one=False, cos=dv(cos),
                        sin=dv(sin), rot=d if rope else 0, interleaved=False, k_cache=k1, v_cache=v1,
                        slots=dev(slots) if write else None, page_size=page)
    for splits in (None, 1, 4, 8, 32):                      # one block a (request, kv head); two and eight, merged by the last
        want = ops.attention_mfma(q1, k1, v1, dev(positions), dev(cu), dev(table), max_q_len=1, max_kv_len=max(lens),
                                  window=window, scale=scale, splits=splits).float().cpu()
        k2, v2 = dev(kc), dev(vc)
        if not write:                                       # a layer that reads another's cache: the new key is there already
            k2.copy_(k1); v2.copy_(v1)
        got = ops.attention_decode_fused(dev(qkv), k2, v2, dev(positions), dev(cu), dev(table), nq=nq, nkv=nkv, d=d,
                                         slots=dev(slots) if write else None, q_norm_w=dv(qw), k_norm_w=dv(kw), eps=1e-5,
                                         add_one=False, cos=dv(cos), sin=dv(sin), max_kv_len=max(lens), window=window,
                                         scale=scale, splits=splits).float().cpu()
        close(got, want, 2 ** -7, f"fused splits={splits}")
        if write:
            assert torch.equal(v2, v1)
            # keys: the same but for a last bit here and there (the sum of squares is added up in another order)
            dk = (k2.float() - k1.float()).abs()
            assert float(dk.max()) <= 2 ** -7 * float(k1.float().abs().max()) and float((dk > 0).float().mean()) < 1e-3
        # the counters that tell the last block are zero again
        counters = ops._DECODE_COUNTERS.get(torch.cuda.current_device())
        assert counters is None or int(counters.abs().sum()) == 0


def test_attention_decode_merge_is_the_same_every_time():
    """The blocks of a (request, key/value head) finish in any order and the last one merges: the sum runs in the
    order of the splits, so twenty calls give the same bits, and so does a call captured in a graph and replayed."""
    from inferrs_amd import ops
    nq, nkv, d, page = 8, 2, 128, 16
    lens = [2000, 1500, 700]
    q, kc, vc, positions, token_seq, table = attention_case(torch.bfloat16, nq, nkv, d, page, lens, [1] * len(lens), 29)
    n = len(lens)
    qkv = dev(randn(n, (nq + 2 * nkv) * d, dtype=torch.bfloat16, seed=3))
    cu = dev(torch.arange(n + 1, dtype=torch.int32))
    k, v, pos, tab = dev(kc), dev(vc), dev(positions), dev(table)
    call = lambda: ops.attention_decode_fused(qkv, k, v, pos, cu, tab, nq=nq, nkv=nkv, d=d, slots=None, q_norm_w=None,
                                              k_norm_w=None, eps=1e-6, add_one=False, cos=None, sin=None,
                                              max_kv_len=max(lens), window=None, scale=d ** -0.5, splits=64)
    first = call().clone()
    for _ in range(20):
        assert torch.equal(call(), first)
    want = ops.attention_mfma(qkv[:, :nq * d].view(n, nq, d).contiguous(), k, v, pos, cu, tab, max_q_len=1,
                              max_kv_len=max(lens), window=None, scale=d ** -0.5, splits=1)
    close(first, want.float().cpu(), 2 ** -7, "64 splits against one")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = call()
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, first)
        assert torch.equal(call(), first)                   # eager work between the replays


def test_attention_decode_counters_are_not_made_under_capture():
    """The counters are allocated at a first call outside a graph capture; a capture that would have to allocate
    them says so instead of putting them into the graph's own memory."""
    from inferrs_amd import ops
    nq, nkv, d, page = 4, 1, 64, 16
    lens = [600]
    q, kc, vc, positions, token_seq, table = attention_case(torch.bfloat16, nq, nkv, d, page, lens, [1], 31)
    qkv = dev(randn(1, (nq + 2 * nkv) * d, dtype=torch.bfloat16, seed=4))
    args = (qkv, dev(kc), dev(vc), dev(positions), dev(torch.arange(2, dtype=torch.int32)), dev(table))
    kw = dict(nq=nq, nkv=nkv, d=d, slots=None, q_norm_w=None, k_norm_w=None, eps=1e-6, add_one=False, cos=None, sin=None,
              max_kv_len=600, window=None, scale=d ** -0.5, splits=16)
    kept = dict(ops._DECODE_COUNTERS)
    ops._DECODE_COUNTERS.clear()
    try:
        graph = torch.cuda.CUDAGraph()
        with pytest.raises(ops.KernelError, match="graph capture"):
            with torch.cuda.graph(graph):
                ops.attention_decode_fused(*args, **kw)
        eager = ops.attention_decode_fused(*args, **kw)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = ops.attention_decode_fused(*args, **kw)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
    finally:
        ops._DECODE_COUNTERS.update({k: v for k, v in kept.items() if k not in ops._DECODE_COUNTERS})


# ---- products of 17 to 128 rows (gemm_mid.hip) ----------------------------------------------------------------

@pytest.mark.parametrize("m", [1, 17, 31, 32, 33, 48, 64, 65, 90, 96, 97, 128])
@pytest.mark.parametrize("n,k", [(64, 128), (80, 256), (200, 896), (4096, 1024), (6144, 4096), (77, 3 * 128)])
def test_mid_product(m, n, k):
    """Every number of rows up to 128 (row tiles that are partly empty; beyond 64 rows another pipeline), feature counts that are no multiple of the
    block's 64 or of 4, k ranges of one chunk, of fewer chunks than the pipeline is deep and of many; plain, in 32-bit,
    and split along k."""
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=m)
    w = randn(n, k, dtype=torch.bfloat16, seed=n + k, scale=0.05)
    want = x.float() @ w.float().t()
    close(ops.gemm_mid_bf16(dev(x), dev(w)), want, 2 ** -8, "mid product")
    close(ops.gemm_mid_bf16(dev(x), dev(w), torch.float32), want, 2e-6 * math.sqrt(k), "mid product, 32-bit result")
    split = ops.gemm_mid_bf16(dev(x), dev(w), partial=True)
    if isinstance(split, ops.Partials):
        assert split.parts.shape[0] == ops.library().ia_gemm_mid_splits(n, k) > 1
        close(split.parts.sum(0), want, 2e-6 * math.sqrt(k), "the splits' sums")
        close(split.materialize(), want, 2 ** -8, "sum of the splits")
    else:
        assert ops.library().ia_gemm_mid_splits(n, k) == 1 or (m * n) % 4


def test_mid_product_splits_depend_on_the_weight_alone():
    from inferrs_amd import ops
    lib = ops.library()
    assert lib.ia_gemm_mid_splits(4096, 4096) > 1 and lib.ia_gemm_mid_splits(151936, 4096) == 1
    assert lib.ia_gemm_mid_splits(4096, 100) == 0                    # k that is no multiple of 128 is not taken
    for n, k in ((4096, 4096), (4096, 12288), (6144, 4096), (5120, 25600)):
        s = lib.ia_gemm_mid_splits(n, k)
        assert k % (128 * s) == 0 and k // s >= 512


@pytest.mark.parametrize("m", [17, 40, 64, 70, 128])
@pytest.mark.parametrize("n,k", [(32, 128), (50, 256), (1408, 1024)])
def test_mid_product_with_the_activation_inside(m, n, k):
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=3 * m)
    w = randn(2 * n, k, dtype=torch.bfloat16, seed=n, scale=0.08)
    gate = (x.float() @ w[:n].float().t()).bfloat16().float()
    up = (x.float() @ w[n:].float().t()).bfloat16().float()
    want = gate / (1 + torch.exp(-gate)) * up
    close(ops.gemm_mid_bf16(dev(x), dev(w), dual=True), want, 2 ** -7, "mid product with SiLU")
    close(ops.gated_silu_linear(dev(x), dev(w)), want, 2 ** -7, "gated_silu_linear")


def test_mid_product_rows_do_not_depend_on_the_batch():
    """A row's result is bit for bit the same whatever else is in the step: alone in a tile, among 64 or 128 rows (which
    walk k in other chunks, four stages deep), at another place among them."""
    from inferrs_amd import ops
    k, n = 1024, 4096
    x = randn(128, k, dtype=torch.bfloat16, seed=8)
    w = dev(randn(n, k, dtype=torch.bfloat16, seed=9, scale=0.05))
    whole = ops.gemm_mid_bf16(dev(x), w).cpu()
    wd = dev(randn(2 * 1408, k, dtype=torch.bfloat16, seed=10, scale=0.05))
    whole_gated = ops.gemm_mid_bf16(dev(x), wd, dual=True).cpu()
    for rows in ([5], list(range(17)), [63, 0, 31, 32], list(range(20, 53)), list(range(64)), list(range(30, 110)), [127, 64, 3]):
        assert torch.equal(ops.gemm_mid_bf16(dev(x[rows].contiguous()), wd, dual=True).cpu(), whole_gated[rows]), rows
        part = ops.gemm_mid_bf16(dev(x[rows].contiguous()), w).cpu()
        assert torch.equal(part, whole[rows]), rows
    split = ops.gemm_mid_bf16(dev(x), w, partial=True)
    assert isinstance(split, ops.Partials)
    again = ops.gemm_mid_bf16(dev(x[10:40].contiguous()), w, partial=True)
    assert torch.equal(again.parts.cpu(), split.parts[:, 10:40].cpu())


@pytest.mark.parametrize("m", [5, 33, 64, 83, 128])
def test_mid_product_with_every_shape_of_block(m):
    """The rule picks the waves of a block and the split of k by the weight's shape; here every shape is forced on one
    weight (features that fill no block, rows that fill no tile): plain with its sums split two ways, and with the
    activation inside."""
    from inferrs_amd import ops
    lib = ops.library()
    n, k = 300, 1024
    x = dev(randn(m, k, dtype=torch.bfloat16, seed=1))
    w = dev(randn(n, k, dtype=torch.bfloat16, seed=2, scale=0.05))
    wd = dev(randn(2 * n, k, dtype=torch.bfloat16, seed=3, scale=0.05))
    want = x.float().cpu() @ w.float().cpu().t()
    gate = (x.float().cpu() @ wd[:n].float().cpu().t()).bfloat16().float()
    up = (x.float().cpu() @ wd[n:].float().cpu().t()).bfloat16().float()
    try:
        for waves in range(2, 9):
            lib.ia_gemm_mid_plan(waves, 2, 3)
            assert lib.ia_gemm_mid_splits(n, k) == 2
            parts = ops.gemm_mid_bf16(x, w, partial=True)
            assert isinstance(parts, ops.Partials) and parts.parts.shape[0] == 2
            close(parts.materialize(), want, 2 ** -8, f"{waves} waves a block")
            if waves % 2 == 0:
                lib.ia_gemm_mid_plan(waves, 1, 3)
                close(ops.gemm_mid_bf16(x, wd, dual=True), gate / (1 + torch.exp(-gate)) * up, 2 ** -7,
                      f"{waves} waves a block with SiLU")
        # a shape that has no kernel is refused where it is asked for, and changes nothing
        for bad in ((9, 1, 3), (1, 1, 3), (4, 3, 3), (6, 2, 2), (4, 32, 3)):
            assert lib.ia_gemm_mid_plan(*bad) != 0 and b"gemm_mid_plan" in lib.ia_last_error()
        close(ops.gemm_mid_bf16(x, wd, dual=True), gate / (1 + torch.exp(-gate)) * up, 2 ** -7, "after refused plans")
        # k that does not split into whole chunks for every block: refused by the launcher, never a lost tail
        lib.ia_gemm_mid_plan(4, 16, 3)
        with pytest.raises(ops.KernelError, match="does not split 16 ways"):
            ops.gemm_mid_bf16(x, w, partial=True)
    finally:
        lib.ia_gemm_mid_plan(0, 0, 0)


def test_which_kernels_a_gated_product_of_17_to_64_rows_takes(monkeypatch):
    """[gate; up] at 17 to 64 rows: the kernel with the activation inside up to `MID_DUAL_MAX_BYTES`, the vendor's GEMM
    and the SiLU kernel beyond, never the plain product of 17 to 64 rows with the SiLU kernel behind it; the same
    values either way."""
    from inferrs_amd import ops
    x = dev(randn(32, 512, dtype=torch.bfloat16, seed=1))
    w = dev(randn(2 * 640, 512, dtype=torch.bfloat16, seed=2, scale=0.05))
    def entry_points():
        with ops.KernelTimer() as timer:
            out = ops.gated_silu_linear(x, w)
        return out, set(timer.summary())
    inside, names = entry_points()
    assert names == {"gemm_mid_bf16"}
    monkeypatch.setattr(ops, "MID_DUAL_MAX_BYTES", w.numel() * 2 - 1)
    outside, names = entry_points()
    assert names == {"vendor_gemm", "gate_mul"}
    want = torch.nn.functional.silu(x.float() @ w[:640].float().t()) * (x.float() @ w[640:].float().t())
    close(inside, want.cpu(), 2 ** -6, "activation inside")
    close(outside, want.cpu(), 2 ** -6, "vendor's product and the SiLU kernel")


@pytest.mark.parametrize("cols,add_one", [(128, False), (4096, False), (5120, True), (8192, False)])
def test_add_rmsnorm_of_a_split_product(cols, add_one):
    """The norm kernel that adds up a product's splits equals the plain add-and-norm kernel on the stored product."""
    from inferrs_amd import ops
    rows, splits = 37, 4
    x = randn(rows, cols, dtype=torch.bfloat16, seed=1, scale=2.0)
    parts = randn(splits, rows, cols, dtype=torch.float32, seed=2)
    w = randn(cols, dtype=torch.float32, seed=3)
    stored = ops.Partials(dev(parts)).materialize()
    assert torch.equal(stored.cpu(), parts.sum(0).bfloat16()) or float((stored.cpu().float() - parts.sum(0)).abs().max()) < 0.05
    x1, x2 = dev(x.clone()), dev(x.clone())
    want = ops.add_rmsnorm(x1, stored, dev(w), 1e-5, add_one)
    got = ops.add_rmsnorm_partials(x2, ops.Partials(dev(parts)), dev(w), 1e-5, add_one)
    assert torch.equal(x1.cpu(), x2.cpu())
    close(got, want, 2 ** -8, "add_rmsnorm_partials")


def test_mid_product_is_the_same_for_every_pipeline_shape():
    """Chunks of 64 or 128 k and two to four stages of them in shared memory change when a value arrives, never the
    order of a sum: the results are bit for bit the same, with the activation inside as well, and a row's result is the
    same whatever stands beside it."""
    from inferrs_amd import ops
    lib = ops.library()
    x = dev(randn(50, 2048, dtype=torch.bfloat16, seed=1))
    w = dev(randn(200, 2048, dtype=torch.bfloat16, seed=2, scale=0.05))
    wd = dev(randn(2 * 96, 2048, dtype=torch.bfloat16, seed=3, scale=0.05))
    try:
        outs = {}
        for kc, ns in ((0, 0), (4, 2), (4, 3), (2, 3), (2, 4)):
            lib.ia_gemm_mid_tune(kc, ns)
            outs[(kc, ns)] = (ops.gemm_mid_bf16(x, w).cpu(), ops.gemm_mid_bf16(x, wd, dual=True).cpu(),
                              ops.gemm_mid_bf16(x[7:30].contiguous(), wd, dual=True).cpu(),
                              ops.gemm_mid_bf16(x[:32].contiguous(), wd, dual=True).cpu())
        assert lib.ia_gemm_mid_tune(8, 2) != 0 and b"gemm_mid_tune" in lib.ia_last_error()
        assert torch.equal(ops.gemm_mid_bf16(x, w).cpu(), outs[(2, 4)][0])          # the refused pipeline changed nothing
    finally:
        lib.ia_gemm_mid_tune(0, 0)
    first = outs[(0, 0)]
    assert all(torch.equal(o[0], first[0]) and torch.equal(o[1], first[1]) for o in outs.values())
    assert all(torch.equal(o[2], o[3][7:30]) and torch.equal(o[2], o[1][7:30]) for o in outs.values())
    gate = (x.float().cpu() @ wd[:96].float().cpu().t()).bfloat16().float()
    up = (x.float().cpu() @ wd[96:].float().cpu().t()).bfloat16().float()
    for o in outs.values():
        close(o[0], x.float().cpu() @ w.float().cpu().t(), 2 ** -8, "mid product")
        close(o[1], gate / (1 + torch.exp(-gate)) * up, 2 ** -7, "mid product with SiLU")


@pytest.mark.parametrize("m", [20, 50, 64, 83, 96, 128])
def test_mid_product_is_the_same_however_the_waves_share_a_block(m):
    """A wave takes one tile of weight rows over all rows of the step, or two tiles (with the activation inside: the gate
    rows and the up rows of the same features) over half of the rows: fewer operand reads, the same sums in the same
    order.  Bit for bit, plain, split along k and with the activation inside, with features that fill no pair of tiles, for
    every even number of waves."""
    from inferrs_amd import ops
    lib = ops.library()
    n, k = 300, 1024
    x = dev(randn(m, k, dtype=torch.bfloat16, seed=11))
    w = dev(randn(n, k, dtype=torch.bfloat16, seed=12, scale=0.05))
    wd = dev(randn(2 * n, k, dtype=torch.bfloat16, seed=13, scale=0.05))
    try:
        for waves in (0, 2, 4, 6, 8):
            outs = []
            for how in (1, 2):
                assert lib.ia_gemm_mid_blocking(how) == 0
                if waves:
                    lib.ia_gemm_mid_plan(waves, 2, 3)
                split = ops.gemm_mid_bf16(x, w, partial=True)
                if waves:
                    lib.ia_gemm_mid_plan(waves, 1, 3)
                outs.append((split.parts.cpu() if isinstance(split, ops.Partials) else split.cpu(),
                             ops.gemm_mid_bf16(x, w, torch.float32).cpu() if not waves else None,
                             ops.gemm_mid_bf16(x, wd, dual=True).cpu()))
            for a, b in zip(*outs):
                assert a is None or torch.equal(a, b), (waves, m)
        assert lib.ia_gemm_mid_blocking(3) != 0 and b"gemm_mid_blocking" in lib.ia_last_error()
    finally:
        lib.ia_gemm_mid_plan(0, 0, 0)
        lib.ia_gemm_mid_blocking(0)
    gate = (x.float().cpu() @ wd[:n].float().cpu().t()).bfloat16().float()
    up = (x.float().cpu() @ wd[n:].float().cpu().t()).bfloat16().float()
    close(outs[1][2], gate / (1 + torch.exp(-gate)) * up, 2 ** -7, "pairs of tiles with SiLU")


def _gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gate_mul_with_gelu(dtype):
    """The gate's activation is a parameter of the kernel: GELU in its tanh form against torch's own."""
    from inferrs_amd import ops
    gu = randn(5, 2 * 203, dtype=dtype, seed=4, scale=4.0)
    g, u = gu[:, :203].float(), gu[:, 203:].float()
    close(ops.gate_mul(dev(gu), "gelu_tanh"), torch.nn.functional.gelu(g, approximate="tanh") * u, tol(dtype), "gate_mul gelu")
    close(ops.gate_mul(dev(gu), "gelu_tanh"), _gelu_tanh(g.double()) * u.double(), tol(dtype), "gate_mul gelu, written out")
    close(ops.gate_mul(dev(gu), "silu"), torch.nn.functional.silu(g) * u, tol(dtype), "gate_mul silu")
    with pytest.raises(ops.KernelError, match="relu"):
        ops.gate_mul(dev(gu), "relu")


@pytest.mark.parametrize("m", [1, 8, 17, 40, 64, 300])
@pytest.mark.parametrize("n,k", [(130, 40), (1536, 512), (200, 136), (12288, 512)])
def test_gated_linear_with_gelu(m, n, k, monkeypatch):
    """Every product that has the gate's activation inside (few rows, 17 to 64 rows, few rows on blocks that fill the
    chip, the tiled product of many rows) takes GELU as it takes SiLU."""
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=1)
    w = randn(2 * n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    gate = (x.double() @ w[:n].double().t()).to(torch.bfloat16).double()
    up = (x.double() @ w[n:].double().t()).to(torch.bfloat16).double()
    want = _gelu_tanh(gate) * up
    close(ops.gated_linear(dev(x), dev(w), "gelu_tanh"), want, 2 ** -7, "fused")
    if m > 64 and k % 64 == 0:
        monkeypatch.setattr(ops, "LARGE_PRODUCTS", "own")
        with ops.KernelTimer() as timer:
            got = ops.gated_linear(dev(x), dev(w), "gelu_tanh")
        assert set(timer.summary()) == {"gemm_mfma_bf16"}
        close(got, want, 2 ** -7, "tiled product")


@pytest.mark.parametrize("m", [1, 5, 16, 17, 50, 200])
@pytest.mark.parametrize("n,k", [(130, 40), (1536, 512), (4096, 1024), (200, 136)])
def test_products_with_a_bias(m, n, k):
    """x . w^T + b for every row count: inside the skinny product's sums (up to 16 rows), behind every other product
    by the kernel that adds a row to all rows; 32-bit results and 32-bit operands too."""
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=1)
    w = randn(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    b = randn(n, dtype=torch.bfloat16, seed=3, scale=3.0)
    want = x.double() @ w.double().t() + b.double()
    close(ops.linear(dev(x), dev(w), bias=dev(b)), want, 2 ** -7, "bfloat16")
    out32 = ops.linear(dev(x), dev(w), torch.float32, bias=dev(b))
    assert out32.dtype == torch.float32
    close(out32, want, 2e-5 if m <= 16 else 2 ** -7, "32-bit result")
    close(ops.linear(dev(x.float()), dev(w.float()), bias=dev(b.float())), want, 2e-6, "32-bit operands")
    with pytest.raises(ops.KernelError, match="bias"):
        ops.linear(dev(x), dev(w), bias=dev(b[:-1].contiguous()))
    # [gate; up] with a bias on both halves, before the activation
    w2 = randn(2 * n, k, dtype=torch.bfloat16, seed=4, scale=0.05)
    b2 = randn(2 * n, dtype=torch.bfloat16, seed=5, scale=0.5)
    full = x.double() @ w2.double().t() + b2.double()
    if m <= 16:                 # in the sums, rounded once
        gate, up = full[:, :n].to(torch.bfloat16).double(), full[:, n:].to(torch.bfloat16).double()
        close(ops.gated_linear(dev(x), dev(w2), "silu", dev(b2)), gate / (1 + torch.exp(-gate)) * up, 2 ** -7, "gated, few rows")
    else:                       # behind the stored product
        close(ops.gated_linear(dev(x), dev(w2), "gelu_tanh", dev(b2)), _gelu_tanh(full[:, :n]) * full[:, n:], 2 ** -6, "gated")


@pytest.mark.parametrize("m", [1, 8, 16])
@pytest.mark.parametrize("n,k,add_one", [(4096, 1024, False), (520, 256, True), (200, 40, False)])
def test_a_product_with_a_bias_adds_itself_to_the_stream(m, n, k, add_one):
    """The product that adds itself to the residual stream takes a bias along: the stream holds what the add kernel
    would leave of the stored product with the bias in it, and the sums of squares and scaled rows are those of
    the new rows; the product that finishes a norm takes one as well."""
    from inferrs_amd import ops
    x = randn(m, k, dtype=torch.bfloat16, seed=31)
    w = randn(n, k, dtype=torch.bfloat16, seed=32, scale=0.03)
    b = randn(n, dtype=torch.bfloat16, seed=37, scale=2.0)
    stream = randn(m, n, dtype=torch.bfloat16, seed=33)
    norm_w = (0.0 if add_one else 1.0) + 0.1 * randn(n, dtype=torch.float32, seed=34)
    plain_stream = dev(stream)
    plain_rows = ops.add_rmsnorm(plain_stream, ops.gemm_skinny_bf16(dev(x), dev(w), bias=dev(b)), dev(norm_w), 1e-6, add_one)
    fused_stream = dev(stream)
    norm = _Norm(dev(norm_w), add_one)
    sums, scaled = ops.linear_add(dev(x), dev(w), fused_stream, norm, dev(b))
    assert torch.equal(fused_stream, plain_stream), "the stream after the sum"
    product = (x.double() @ w.double().t() + b.double()).to(torch.bfloat16)           # (the bias is in before the rounding)
    close(fused_stream, product.double() + stream.double(), 2 ** -7, "the stream against the sum written out")
    rows = ops.NormedRows(fused_stream, scaled, sums, norm.weight, 1e-6, add_one)
    assert torch.equal(rows.materialize(), plain_rows)
    n2 = 264
    w2 = randn(n2, n, dtype=torch.bfloat16, seed=35, scale=0.03)
    b2 = randn(n2, dtype=torch.bfloat16, seed=38, scale=2.0)
    new_rows = fused_stream.float().cpu().double()
    exact = new_rows / torch.sqrt(new_rows.pow(2).mean(-1, keepdim=True) + 1e-6) * (norm_w.double() + (1.0 if add_one else 0.0))
    close(ops.linear(rows, dev(w2), bias=dev(b2)), exact @ w2.double().t() + b2.double(), 2 ** -6, "norm's end and bias inside")


@pytest.mark.parametrize("dtype", DTYPES)
def test_few_row_product_of_the_32_bit_path_with_every_block_shape(dtype):
    """The product for up to 16 rows with 4, 8 or 16 output features and 8 or 16 staged rows a wave (100 * features +
    rows names a shape; one that does not hold the rows gives way to one that does): one chain of fused multiply-adds
    for every output in all of them, so the bits are the same, and those of the tiled kernel that takes more rows."""
    from inferrs_amd import ops
    lib = ops.library()
    x = randn(80, 520, dtype=dtype, seed=1)
    w = dev(randn(203, 520, dtype=dtype, seed=2, scale=0.05))
    many = ops.gemm_tiled(dev(x), w).cpu()                      # 80 rows: tiles of 64 x 64
    outs = {}
    try:
        for features in (816, 808, 416, 1608, 0):
            assert lib.ia_gemm_rows_tune(features) == 0
            outs[features] = [ops.gemm_tiled(dev(x[:m].contiguous()), w).cpu() for m in (1, 7, 8, 9, 16)]
        assert lib.ia_gemm_rows_tune(1616) != 0 and "16 features and 16 rows" in lib.ia_last_error().decode()
    finally:
        lib.ia_gemm_rows_tune(0)
    for features, got in outs.items():
        for i, y in enumerate(got):
            assert torch.equal(y, outs[816][i]), (features, i)
            if dtype == torch.float32:
                assert torch.equal(y, many[:y.shape[0]]), (features, y.shape)
            close(y, x[:y.shape[0]].double() @ w.double().cpu().t(), tol(dtype, 2e-6), "few rows")


@pytest.mark.parametrize("m,n,k", [(130, 72, 40), (512, 4096, 1024), (2048, 6144, 4096), (300, 1000, 136), (129, 64, 33), (1024, 1024, 3072)])
def test_vendor_gemm_called_directly_is_the_product_that_torch_gets(m, n, k):
    """The vendor's GEMM through this package's own entry point (descriptors and the library's choice of kernel kept
    for every shape) against the exact product and against the same library through torch; a shape that the
    library's search has no kernel for goes through torch and is remembered."""
    from inferrs_amd import ops
    x, w = randn(m, k, dtype=torch.bfloat16, seed=1), randn(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    assert ops.VENDOR_GEMM == "direct"
    got = ops.vendor_gemm_bf16(dev(x), dev(w))
    assert ops.library().ia_vendor_gemm_ready() == 1
    again = ops.vendor_gemm_bf16(dev(x), dev(w))                    # the kept plan
    assert torch.equal(got, again)
    close(got, x.double() @ w.double().t(), 2 ** -7, "vendor's product")
    through_torch = torch.nn.functional.linear(dev(x), dev(w))
    close(got, through_torch.float().cpu(), 2 ** -7, "the two ways to the library")
