"""Each HIP kernel alone against its plain PyTorch statement (ops/reference.py), at sizes
other than the engine tests' models: widths and vocabularies that are no power of two,
head sizes in steps of 16, odd head counts and groups."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DT = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from jax_llm_examples_amd.engine import get_ops
    return get_ops(DEV)


@pytest.fixture(scope="module")
def ref():
    from jax_llm_examples_amd.ops.reference import ReferenceOps
    return ReferenceOps()


def _tol(dt):
    return dict(rtol=2e-5, atol=2e-6) if dt == torch.float32 else dict(rtol=1.6e-2, atol=1e-3)


def _assert_close_to_scale(got, want, dt):
    """For results that are sums of many rounded terms: error against the size of the whole result."""
    tol = 2e-5 if dt == torch.float32 else 1e-2
    err = float((got.float() - want.float()).abs().max() / want.float().abs().max())
    assert err <= tol, f"error {err:.3g} of the largest value, allowed {tol}"


def _rand(*shape, dt=torch.float32, scale=1.0, seed=None):
    g = torch.Generator(device="cpu").manual_seed(seed if seed is not None else hash(shape) % 1000)
    return (torch.randn(*shape, generator=g) * scale).to(dt).to(DEV)


@pytest.mark.parametrize("dt", DT)
def test_embed(ops, ref, dt):
    table = _rand(311, 80, dt=dt)
    tok = torch.tensor([0, 310, 5, 5, 17], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.embed(tok, table), ref.embed(tok, table))


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("d", [80, 1000, 1026, 1028, 2056, 5120, 8192, 9000])
def test_add_rmsnorm(ops, ref, dt, d):
    for delta_dt, weighted, want32 in [(None, True, False), (dt, True, True), (torch.float32, False, True)]:
        x = _rand(7, d, seed=1)
        delta = None if delta_dt is None else _rand(7, d, dt=delta_dt, seed=2)
        w = _rand(d, seed=3) if weighted else None
        x1, x2 = x.clone(), x.clone()
        h1, h32_1 = ops.add_rmsnorm(x1, delta, w, 1e-3, dt, want32)
        h2, h32_2 = ref.add_rmsnorm(x2, delta, w, 1e-3, dt, want32)
        assert torch.allclose(x1, x2, rtol=1e-6, atol=1e-6)  # the residual is updated in place, float32
        assert torch.allclose(h1.float(), h2.float(), **_tol(dt))
        if want32:
            assert torch.allclose(h32_1, h32_2, rtol=2e-5, atol=2e-6)
            assert h32_1.dtype == torch.float32


def test_rmsnorm_eps_is_inside_the_root(ops):
    x = torch.full((1, 64), 1e-3, device=DEV)
    h, _ = ops.add_rmsnorm(x, None, None, 1e-2, torch.float32)
    assert torch.allclose(h, torch.full_like(h, 1e-3 / math.sqrt(1e-6 + 1e-2)), rtol=1e-5)


@pytest.mark.parametrize("dt", DT)
def test_silu_mul_gather_add(ops, ref, dt):
    for f in (56, 52, 1000):  # halves that are 16-byte aligned (8 elements per thread in bfloat16), and not
        gu = _rand(9, 2 * f, dt=dt, scale=3.0)
        assert torch.allclose(ops.silu_mul(gu).float(), ref.silu_mul(gu).float(), **_tol(dt))
    x = _rand(11, 90, dt=dt)
    idx = torch.tensor([10, 0, 3, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.gather_rows(x, idx), x[idx.long()])
    r, d = _rand(11, 90, seed=4), _rand(11, 90, dt=dt, seed=5)
    want = r + d.float()
    ops.add_residual(r, d)
    assert torch.allclose(r, want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dt", DT)
def test_qk_prepare_of_a_token_does_not_depend_on_the_batch(ops, ref, dt):
    """Many tokens take wavefronts that go through several heads each; the results must be those of a token
    prepared alone, bit for bit."""
    hq, hk, dh, n, ps = 40, 8, 128, 320, 16
    qkv, pos, pages, slots, inv_freq = _prep_case(hq, hk, dh, n, ps, dt)
    c1 = torch.zeros(pages, 2, hk, ps, dh, dtype=dt, device=DEV)
    c2, c3 = c1.clone(), c1.clone()
    q1 = ops.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv_freq, 1e-5, (16.0, 0.1)), c1, slots)
    q2 = ref.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv_freq, 1e-5, (16.0, 0.1)), c2, slots)
    assert torch.allclose(q1.float(), q2.float(), **_tol(dt)) and torch.allclose(c1.float(), c2.float(), **_tol(dt))
    few = slice(100, 107)
    q3 = ops.qk_prepare_kv_write(qkv[few].contiguous(), hq, hk, dh, pos[few].contiguous(),
                                 _prep(inv_freq, 1e-5, (16.0, 0.1)), c3, slots[few].contiguous())
    assert torch.equal(q3, q1[few])
    written = c3 != 0
    assert written.any() and torch.equal(c3[written], c1[written])


def _prep(inv_freq=None, eps=None, qs=None, **kw):
    from jax_llm_examples_amd.parts.base import QKPreparation, Rotation

    rot = None if inv_freq is None else Rotation(inv_freq, kw.pop("pairing", "adjacent"), kw.pop("rotary_dim", 0))
    return QKPreparation(rotation=rot, norm_eps=eps, query_scale=qs, **kw)


def _prep_case(hq, hk, dh, n, ps, dt, seed=0):
    qkv = _rand(n, (hq + 2 * hk) * dh, dt=dt, seed=seed)
    pos = torch.randint(0, 500, (n,), generator=torch.Generator().manual_seed(seed)).to(torch.int32).to(DEV)
    pages = 2 * n // ps + 3
    slots = torch.randperm(pages * ps, generator=torch.Generator().manual_seed(seed + 1))[:n].to(torch.int32).to(DEV)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, dh, 2).float() / dh))).to(DEV)
    return qkv, pos, pages, slots, inv_freq


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("hq,hk,dh", [(4, 2, 16), (5, 1, 48), (40, 8, 128), (3, 3, 256), (6, 2, 80)])
def test_qk_prepare_kv_write(ops, ref, dt, hq, hk, dh):
    n, ps = 13, 8
    qkv, pos, pages, slots, inv_freq = _prep_case(hq, hk, dh, n, ps, dt)
    for rope, eps, qs in [(True, 1e-5, None), (False, None, (16.0, 0.1)), (True, None, None), (False, None, None),
                          (True, 1e-3, (4.0, 0.3))]:
        c1 = torch.zeros(pages, 2, hk, ps, dh, dtype=dt, device=DEV)
        c2 = c1.clone()
        q1 = ops.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv_freq if rope else None, eps, qs), c1, slots)
        q2 = ref.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv_freq if rope else None, eps, qs), c2, slots)
        assert torch.allclose(q1.float(), q2.float(), **_tol(dt))
        assert torch.allclose(c1.float(), c2.float(), **_tol(dt))
        assert (c1[:, 1] != 0).any() and torch.equal(c1 == 0, c2 == 0)  # wrote exactly the same places
    q3 = ops.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv_freq), None, None)  # a run that only reads
    assert torch.allclose(q3.float(), ref.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv_freq), None,
                                                               None).float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("hq,hk,dh,rd", [(4, 2, 32, 32), (5, 1, 48, 16), (40, 8, 128, 64), (6, 2, 80, 80)])
def test_qk_prepare_other_rotations_and_norms(ops, ref, dt, hq, hk, dh, rd):
    """What Llama 4 does not use but the preparation takes as data: half-split pairs, a rotation of the
    head's leading part only, norm weights, the norm before the rotation."""
    n, ps = 11, 8
    qkv, pos, pages, slots, _ = _prep_case(hq, hk, dh, n, ps, dt, seed=3)
    inv = (1.0 / (10000.0 ** (torch.arange(0, rd, 2).float() / rd))).to(DEV)
    wq, wk = _rand(dh, seed=7) + 1.5, _rand(dh, seed=8) - 1.5
    cases = [dict(pairing="half", rotary_dim=rd), dict(pairing="adjacent", rotary_dim=rd),
             dict(pairing="half", rotary_dim=rd, eps=1e-4, norm_weight_q=wq, norm_weight_k=wk),
             dict(pairing="adjacent", rotary_dim=rd, eps=1e-4, norm_weight_q=wq, norm_weight_k=wk, norm_first=True),
             dict(pairing="half", rotary_dim=rd, eps=1e-2, norm_first=True, qs=(4.0, 0.3))]
    for kw in cases:
        c1 = torch.zeros(pages, 2, hk, ps, dh, dtype=dt, device=DEV)
        c2 = c1.clone()
        q1 = ops.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv, **dict(kw)), c1, slots)
        q2 = ref.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv, **dict(kw)), c2, slots)
        assert torch.allclose(q1.float(), q2.float(), **_tol(dt)), kw
        assert torch.allclose(c1.float(), c2.float(), **_tol(dt)), kw
    # the pairing matters: half-split and adjacent pairs give different rows
    a = ref.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv, pairing="half", rotary_dim=rd), None, None)
    b = ref.qk_prepare_kv_write(qkv, hq, hk, dh, pos, _prep(inv, pairing="adjacent", rotary_dim=rd), None, None)
    assert not torch.allclose(a.float(), b.float(), atol=1e-2)


def test_rotation_angles_are_float32_at_large_positions(ops):
    # the angle must be pos * inv_freq in float32: with a bfloat16 position 257 becomes 256
    dh = 16
    qkv = torch.zeros(1, 3 * dh, device=DEV)
    qkv[0, 0] = 1.0
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, dh, 2).float() / dh))).to(DEV)
    for p in (257, 4099, 131071):
        pos = torch.tensor([p], dtype=torch.int32, device=DEV)
        q = ops.qk_prepare_kv_write(qkv, 1, 1, dh, pos, _prep(inv_freq), None, None)
        assert abs(float(q[0, 0, 0]) - math.cos(float(torch.tensor(float(p)) * inv_freq[0].cpu()))) < 2e-6
        assert abs(float(q[0, 0, 1]) - math.sin(float(torch.tensor(float(p)) * inv_freq[0].cpu()))) < 2e-6


def _attention_case(hq, hk, dh, ps, dt, seg_specs, seed=0):
    """seg_specs: (tokens already in the cache, new tokens) per segment; pages are scattered."""
    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(a + b) // ps) for a, b in seg_specs) + 5
    perm = torch.randperm(total_pages, generator=g).tolist()
    kv = (torch.randn(total_pages, 2, hk, ps, dh, generator=g) * 0.7).to(dt).to(DEV)
    width = max(-(-(a + b) // ps) for a, b in seg_specs)
    bt = torch.full((len(seg_specs), width), -1, dtype=torch.int32)
    pos, seg = [], []
    for i, (a, b) in enumerate(seg_specs):
        for j in range(-(-(a + b) // ps)):
            bt[i, j] = perm.pop()
        pos += list(range(a, a + b))
        seg += [i] * b
    n = len(pos)
    q = (torch.randn(n, hq, dh, generator=g)).to(dt).to(DEV)
    return (q, kv, bt.to(DEV), torch.tensor(pos, dtype=torch.int32, device=DEV),
            torch.tensor(seg, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("hq,hk,dh,ps", [(4, 2, 16, 16), (5, 1, 48, 16), (6, 3, 32, 8), (8, 8, 64, 16),
                                         (10, 2, 128, 16), (2, 1, 256, 32), (3, 1, 80, 16), (6, 3, 32, 16),
                                         (40, 8, 128, 16), (20, 1, 96, 48), (4, 4, 256, 16), (5, 5, 64, 64),
                                         (10, 2, 128, 32), (9, 3, 128, 48), (10, 5, 128, 64)])
@pytest.mark.parametrize("retention", [("all",), ("chunk", 24), ("window", 37)])
def test_paged_attention(ops, ref, dt, hq, hk, dh, ps, retention):
    case = _attention_case(hq, hk, dh, ps, dt, [(0, 70), (130, 1), (45, 9), (63, 2), (200, 1), (600, 1), (255, 3)])
    q, kv, bt, pos, seg = case
    got = ops.paged_attention(q, kv, bt, pos, seg, retention, dh ** -0.5)
    want = ref.paged_attention(q, kv, bt, pos, seg, retention, dh ** -0.5)
    _assert_close_to_scale(got, want, dt)


@pytest.mark.parametrize("hq,hk,dh,ps", [(4, 2, 16, 16), (5, 1, 48, 16), (8, 8, 64, 16), (10, 2, 128, 16), (2, 1, 256, 32),
                                         (3, 1, 80, 16), (20, 1, 96, 48), (9, 3, 128, 48), (5, 5, 64, 64)])
@pytest.mark.parametrize("retention", [("all",), ("chunk", 24), ("chunk", 100), ("window", 37)])
def test_float32_attention_of_portions_on_the_float32_matrix_instructions(ops, ref, monkeypatch, hq, hk, dh, ps, retention):
    """Tiles of 16 tokens per wavefront (steps of many tokens in float32 take this kernel): portions that start
    anywhere, single tokens between them, keys of earlier steps; and a token's result does not depend on which
    tile it falls into."""
    monkeypatch.setattr(type(ops), "GENERIC_SPLIT_BELOW", 0)
    specs = [(0, 70), (130, 1), (45, 9), (63, 2), (200, 1), (600, 1), (255, 35)]
    q, kv, bt, pos, seg = _attention_case(hq, hk, dh, ps, torch.float32, specs)
    calls = []
    inner = ops._call
    monkeypatch.setattr(ops, "_call", lambda name, *a: (calls.append(name), inner(name, *a))[1])
    got = ops.paged_attention(q, kv, bt, pos, seg, retention, dh ** -0.5)
    assert calls == ["jle_attention_f32_tiles"]
    want = ref.paged_attention(q, kv, bt, pos, seg, retention, dh ** -0.5)
    _assert_close_to_scale(got, want, torch.float32)
    # the last 20 tokens of the last portion alone (other tiles, an odd start): the same bits
    n = q.shape[0]
    alone = ops.paged_attention(q[n - 20:].contiguous(), kv, bt, pos[n - 20:].contiguous(), seg[n - 20:].contiguous(),
                                retention, dh ** -0.5)
    assert torch.equal(alone, got[n - 20:])


@pytest.mark.parametrize("hq,hk,dh,ps", [(4, 2, 16, 16), (5, 1, 48, 16), (40, 8, 128, 16), (16, 1, 64, 32), (3, 3, 256, 16)])
@pytest.mark.parametrize("retention", [("all",), ("chunk", 100), ("window", 37)])
def test_float32_attention_of_single_tokens_on_the_float32_matrix_instructions(ops, ref, monkeypatch, hq, hk, dh, ps, retention):
    """A step of single tokens in float32: the query heads of a kv head share a wavefront, the keys are shared
    between wavefronts (forced here to ranges of 64 keys, so that every token has several) and merged."""
    monkeypatch.setattr(type(ops), "F32_DECODE_ITEMS", 1 << 20)
    specs = [(130, 1), (0, 1), (63, 1), (200, 1), (600, 1), (15, 1), (99, 1)]
    q, kv, bt, pos, seg = _attention_case(hq, hk, dh, ps, torch.float32, specs)
    calls = []
    inner = ops._call
    monkeypatch.setattr(ops, "_call", lambda name, *a: (calls.append(name), inner(name, *a))[1])
    got = ops.paged_attention(q, kv, bt, pos, seg, retention, dh ** -0.5)
    assert calls == ["jle_attention_f32_heads", "jle_attention_merge"]
    want = ref.paged_attention(q, kv, bt, pos, seg, retention, dh ** -0.5)
    _assert_close_to_scale(got, want, torch.float32)
    monkeypatch.setattr(type(ops), "F32_DECODE_ITEMS", 1)  # one range per token: no merge
    calls.clear()
    whole = ops.paged_attention(q, kv, bt, pos, seg, retention, dh ** -0.5)
    assert calls == ["jle_attention_f32_heads"]
    _assert_close_to_scale(whole, want, torch.float32)


@pytest.mark.parametrize("hq,hk,ps", [(10, 2, 16), (40, 8, 16), (6, 3, 32), (9, 3, 48), (4, 2, 64)])
@pytest.mark.parametrize("retention", [("all",), ("chunk", 192), ("chunk", 100), ("window", 150)])
def test_paged_attention_of_long_portions_at_head_size_128(ops, ref, hq, hk, ps, retention):
    """Portions of hundreds of tokens behind hundreds of cached ones, at the head size whose kernel takes 64 keys a
    step straight into shared memory: many steps, pages of every size crossed inside a step, rules whose first
    key lies inside a step and inside a page."""
    dt = torch.bfloat16
    case = _attention_case(hq, hk, 128, ps, dt, [(0, 333), (190, 130), (517, 1), (64, 64), (1000, 35)], seed=3)
    q, kv, bt, pos, seg = case
    got = ops.paged_attention(q, kv, bt, pos, seg, retention, 128 ** -0.5)
    want = ref.paged_attention(q, kv, bt, pos, seg, retention, 128 ** -0.5)
    _assert_close_to_scale(got, want, dt)


def _decode_case(hq, hk, dh, ps, dt, contexts, seed=0):
    """One new token per request after ``contexts[i]`` tokens in the cache; the step's group context with the
    bound the kernels' work is laid out for; raw q|k|v rows and the slots of the new tokens."""
    from jax_llm_examples_amd.engine.batch import GroupContext, decode_bucket
    q, kv, bt, pos, seg = _attention_case(hq, hk, dh, ps, dt, [(c, 1) for c in contexts], seed=seed)
    n = len(contexts)
    g = torch.Generator().manual_seed(seed + 50)
    qkv = torch.randn(n, (hq + 2 * hk) * dh, generator=g).to(dt).to(DEV)
    slots = torch.tensor([int(bt[i, c // ps]) * ps + c % ps for i, c in enumerate(contexts)], dtype=torch.int32,
                         device=DEV)
    meta = lambda ret: GroupContext(block_table=bt, slot_mapping=slots, width=bt.shape[1], retention=ret,
                                    seg_lens=[1] * n, seg_starts=list(contexts),
                                    decode_bucket=decode_bucket(max(contexts) + 1))
    return qkv, kv, bt, pos, seg, slots, meta


_DECODE_CASES = [
    (40, 8, 128, 16, [3000 + 94 * i for i in range(64)]),  # the serving shape: 64 requests between 3,000 and 9,000
    (40, 8, 128, 16, [8191, 8192, 8193, 0, 5, 16383, 16384, 4095]),
    (10, 2, 64, 32, [0, 1, 31, 32, 700, 129]), (6, 1, 32, 16, [77]), (20, 1, 96, 48, [500, 47, 48]),
    (34, 2, 32, 16, [260, 3]), (4, 4, 256, 16, [90, 1000])]
_DECODE_RETENTIONS = [("all",), ("chunk", 8192), ("chunk", 96), ("window", 200)]


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("hq,hk,dh,ps,contexts,retention",
                         [(*c, r) for c in _DECODE_CASES for r in _DECODE_RETENTIONS
                          if r != ("chunk", 8192) or max(c[4]) >= 3000])  # (the large chunk: long contexts only)
def test_attention_of_a_step_of_single_tokens_from_the_projection_rows(ops, ref, dt, hq, hk, dh, ps, contexts, retention):
    """Rotation, q/k norm, scale, the write of the new key and value, attention over many key ranges and their
    merge: one launch in bfloat16 (two kernels and a merge in float32), against the plain ops."""
    from jax_llm_examples_amd.ops.hip import HipOps
    qkv, kv, bt, pos, seg, slots, meta = _decode_case(hq, hk, dh, ps, dt, contexts)
    inv = (1.0 / (10000.0 ** (torch.arange(0, dh, 2).float() / dh))).to(DEV)
    for prep in (_prep(inv, 1e-5, None), _prep(None, None, (64.0, 0.2)), _prep(inv, None, None)):
        kv1, kv2 = kv.clone(), kv.clone()
        calls = []
        inner = ops._call
        ops._call = lambda name, *a: (calls.append(name), inner(name, *a))[1]
        try:
            got = ops.attention_from_qkv(qkv, hq, hk, dh, pos, seg, prep, kv1, True, slots, bt, retention,
                                         dh ** -0.5, meta(retention))
        finally:
            ops._call = inner
        if dt == torch.bfloat16:
            assert calls == ["jle_attention_decode_fused"], calls
        want = ref.attention_from_qkv(qkv, hq, hk, dh, pos, seg, prep, kv2, True, slots, bt, retention, dh ** -0.5)
        _assert_close_to_scale(got, want, dt)
        assert torch.allclose(kv1.float(), kv2.float(), **_tol(dt))  # the new keys and values are in their pages
        assert int(ops._tickets.abs().sum()) == 0  # the counters are back at zero
        # a run that only reads another run's cache writes nothing
        kv3 = kv2.clone()
        got3 = ops.attention_from_qkv(qkv, hq, hk, dh, pos, seg, prep, kv3, False, slots, bt, retention,
                                      dh ** -0.5, meta(retention))
        assert torch.equal(kv3, kv2)
        _assert_close_to_scale(got3, want, dt)


@pytest.mark.parametrize("dt", DT)
def test_decode_attention_finds_a_far_key_in_every_key_range_and_at_the_chunk_edge(ops, dt):
    """Eight requests around 8,200 tokens: so many key ranges that the work list is longer than the GPU takes at
    once.  One key's score stands out; the output is its value exactly where the rule lets the query see it."""
    hq, hk, dh, ps = 40, 8, 128, 16
    contexts = [8190 + i for i in range(8)]  # positions 8190 .. 8197
    qkv, kv, bt, pos, seg, slots, meta = _decode_case(hq, hk, dh, ps, dt, contexts, seed=2)
    qkv.zero_()
    qkv[:, : hq * dh].view(len(contexts), hq, dh)[:, :, 0] = 8.0  # every query looks along element 0
    prep = _prep(None, None, None)
    kv[:, 0] *= 0.05
    kv[:, 0, :, :, 0] = 0.0

    def run(hot, retention):
        k = kv.clone()
        for i in range(len(contexts)):
            page, off = int(bt[i, hot // ps]), hot % ps
            k[page, 0, :, off, 0] = 8.0
            k[page, 1].view(hk, dh, ps)[:, :, off] = 3.0
        out = ops.attention_from_qkv(qkv, hq, hk, dh, pos, seg, prep, k, False, slots, bt, retention, 1.0,
                                     meta(retention))
        return [bool(v > 2.9) for v in out.float().abs().amin(dim=-1).tolist()]

    for hot in (0, 127, 128, 511, 512, 4100, 8063, 8189):  # first and last range, range edges
        assert run(hot, ("all",)) == [True] * 8, hot
    assert run(8191, ("all",)) == [c >= 8191 for c in contexts]  # causal
    assert run(8191, ("chunk", 8192)) == [c == 8191 for c in contexts]  # the last key of the first chunk
    assert run(8192, ("chunk", 8192)) == [c >= 8192 for c in contexts]  # the first key of the second
    assert run(8000, ("chunk", 8192)) == [c < 8192 for c in contexts]
    assert run(8190 - 299, ("window", 300)) == [c == 8190 for c in contexts]


def test_attention_refuses_a_head_size_it_cannot_do(ops):
    from jax_llm_examples_amd.ops.hip import KernelError
    q, kv, bt, pos, seg = _attention_case(2, 1, 20, 16, torch.float32, [(0, 4)])
    with pytest.raises(KernelError, match="head size 20 is not supported"):
        ops.paged_attention(q, kv, bt, pos, seg, ("all",), 1.0)
    with pytest.raises(KernelError, match="top_k 9"):
        ops.moe_route(torch.zeros(2, 64, device=DEV), torch.zeros(16, 64, device=DEV), 9)


@pytest.mark.parametrize("dt", DT)
def test_attention_finds_one_far_key_among_hundreds_and_respects_the_window_edge(ops, dt):
    """Random weights would hide a key that is skipped: here one key's score stands out, so the
    output is that key's value, if and only if the rule lets the query see it."""
    hq, hk, dh, ps = 2, 1, 32, 16
    T = 700
    q, kv, bt, pos, seg = _attention_case(hq, hk, dh, ps, dt, [(T - 1, 1)], seed=3)
    q.zero_()
    q[0, :, 0] = 8.0

    def run(hot, retention):
        k = kv.clone()
        k[:, 0] *= 0.05
        page, off = int(bt[0, hot // ps]), hot % ps
        k[page, 0, 0, off, 0] = 8.0  # score 64 * scale, far above the rest
        k[page, 1, 0].view(dh, ps)[:, off] = 3.0  # its value (values lie transposed in the page)
        return ops.paged_attention(q, k, bt, pos, seg, retention, 1.0).float()

    for hot in (3, 15, 16, 17, 333, T - 2):  # page edges among them
        assert torch.allclose(run(hot, ("all",)), torch.full((1, hq * dh), 3.0, device=DEV), atol=2e-2)
    C = 96  # the query at 699 is in the chunk that starts at 672
    assert torch.allclose(run(672, ("chunk", C)), torch.full((1, hq * dh), 3.0, device=DEV), atol=2e-2)
    assert run(671, ("chunk", C)).abs().max() < 1.0  # one before the chunk: not seen
    W = 100  # window: keys 600..699
    assert torch.allclose(run(600, ("window", W)), torch.full((1, hq * dh), 3.0, device=DEV), atol=2e-2)
    assert run(599, ("window", W)).abs().max() < 1.0


@pytest.mark.parametrize("dt", DT)
def test_attention_portion_sees_a_far_key_exactly_where_the_rule_allows(ops, dt):
    """The same with a portion of 40 tokens (positions 660..699) in one step: with a chunk of 96 the tokens
    before 672 are in the chunk that starts at 576, the others in the one that starts at 672; with a window
    of 100 each token has its own edge."""
    hq, hk, dh, ps = 4, 2, 32, 16
    q, kv, bt, pos, seg = _attention_case(hq, hk, dh, ps, dt, [(660, 40)], seed=4)
    q.zero_()
    q[:, :, 0] = 8.0

    def run(hot, retention):
        k = kv.clone()
        k[:, 0] *= 0.05
        page, off = int(bt[0, hot // ps]), hot % ps
        k[page, 0, :, off, 0] = 8.0
        k[page, 1].view(hk, dh, ps)[:, :, off] = 3.0
        return ops.paged_attention(q, k, bt, pos, seg, retention, 1.0).float().abs().amin(dim=-1)  # per token

    def sees(out):
        return [bool(v > 2.9) for v in out.tolist()]

    assert sees(run(5, ("all",))) == [True] * 40
    assert sees(run(576, ("chunk", 96))) == [p < 672 for p in range(660, 700)]
    assert sees(run(575, ("chunk", 96))) == [False] * 40
    assert sees(run(672, ("chunk", 96))) == [p >= 672 for p in range(660, 700)]  # causal: not before its own position
    assert sees(run(580, ("window", 100))) == [p - 99 <= 580 for p in range(660, 700)]


def test_attention_reading_a_page_that_was_given_back_is_not_silent(ops):
    q, kv, bt, pos, seg = _attention_case(2, 1, 16, 16, torch.float32, [(40, 1)])
    bt[0, 1] = -1
    out = ops.paged_attention(q, kv, bt, pos, seg, ("all",), 1.0)
    assert torch.isnan(out).all()


@pytest.mark.parametrize("n,d,e,k", [(50, 5120, 16, 1), (7, 80, 3, 2), (33, 96, 128, 4), (1, 64, 4, 1), (70, 50, 5, 2),
                                     (300, 264, 16, 1)])
def test_moe_route(ops, ref, n, d, e, k):
    h, w = _rand(n, d, seed=1), _rand(e, d, scale=0.05, seed=2)
    ids, gates, logits = ops.moe_route(h, w, k, want_logits=True)
    rid, rg = ref.moe_route(h, w, k)
    assert torch.allclose(logits, h @ w.t(), rtol=1e-4, atol=1e-5)
    assert torch.equal(ids, rid) and torch.allclose(gates, rg, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("n,d,e,k,delta", [(1, 5120, 16, 1, "experts"), (8, 5120, 16, 1, "experts"), (64, 5120, 128, 1, "plain"),
                                           (1, 5120, 128, 1, "experts"), (64, 5120, 128, 1, "experts"), (256, 5120, 128, 2, "experts"),
                                           (5, 1032, 3, 2, "plain"), (256, 2048, 37, 4, "none"), (3, 8192, 5, 5, "experts")])
def test_norm_and_router_in_one_launch_equal_the_separate_kernels(ops, dt, n, d, e, k, delta):
    """Addition, norm, router logits, choice and grouping fused for steps of few tokens: bit for bit what the norm
    kernel, the logits kernel and the choose-and-group kernel give one after the other."""
    from jax_llm_examples_amd.ops.hip import ExpertSum
    x = _rand(n, d, seed=1)
    w = _rand(d, seed=2) + 1.0
    router = _rand(e, d, scale=0.05, seed=3)
    if delta == "experts":
        m = n * 2
        routed = _rand(m, d, dt=dt, seed=4)
        inv = torch.randperm(m, generator=torch.Generator().manual_seed(5))[: n * 2].to(torch.int32).to(DEV)
        dl = lambda: ExpertSum(routed, inv, 2, _rand(n, d, dt=dt, seed=6), n, d)
    elif delta == "plain":
        dl = lambda: _rand(n, d, dt=dt, seed=4)
    else:
        dl = lambda: None
    x1, x2 = x.clone(), x.clone()
    h_a, h32_a = ops.add_rmsnorm(x1, dl(), w, 1e-5, dt, want32=True)
    ids_a, gates_a, logits_a, group_a = ops.moe_route(h32_a, router, k, want_logits=True, group=True)
    pending = ops.defer_norm(x2, dl(), w, 1e-5, dt)
    calls = []
    inner = ops._call
    ops._call = lambda name, *a: (calls.append(name), inner(name, *a))[1]
    try:
        ids_b, gates_b, logits_b, group_b = ops.moe_route(pending, router, k, want_logits=True, group=True)
    finally:
        ops._call = inner
    assert calls == ["jle_norm_route"], calls
    assert torch.equal(x2, x)  # the residual is not changed in place: its new value is another tensor
    assert torch.equal(pending.residual(), x1) and torch.equal(pending.rows(), h_a)
    assert torch.equal(logits_b, logits_a) and torch.equal(ids_b, ids_a) and torch.equal(gates_b, gates_a)
    for a, b in zip(group_a, group_b):
        assert torch.equal(a, b)
    assert int(ops._tickets.abs().sum()) == 0
    # sizes the fused kernel does not take go through the separate kernels, with the same results
    wide = ops.defer_norm(_rand(2, 520, seed=1), None, None, 1e-5, dt)
    ids_c, _, _ = ops.moe_route(wide, _rand(4, 520, seed=2), 1, group=True)
    assert wide.done and ids_c.shape == (2, 1)


@pytest.mark.parametrize("n,d,e,k", [(700, 320, 16, 1), (600, 90, 6, 2), (520, 64, 37, 3),
                                     # pieces of 4 x 4, 8 x 4 and 8 x 8 (tokens x experts) per wavefront
                                     (2100, 264, 40, 2), (4100, 520, 24, 1), (4099, 136, 70, 3), (2053, 5120, 128, 1)])
def test_router_logits_of_a_token_do_not_depend_on_the_batch(ops, n, d, e, k):
    """Many rows take other kernel shapes than few (larger pieces per wavefront the more rows and experts there
    are); the sums must come out bit for bit the same, or a token's experts would depend on what else is in the
    step."""
    h, w = _rand(n, d, seed=1), _rand(e, d, scale=0.05, seed=2)
    ids, gates, logits = ops.moe_route(h, w, k, want_logits=True)
    # (against the float64 product: a float32 library product is itself off by about as much as the kernel)
    assert torch.allclose(logits.double(), h.double() @ w.double().t(), rtol=1e-4, atol=1e-5)
    for lo, hi in [(0, 1), (n - 1, n), (100, 107), (3, 300)]:
        i2, g2, l2 = ops.moe_route(h[lo:hi].contiguous(), w, k, want_logits=True)
        assert torch.equal(l2, logits[lo:hi]) and torch.equal(i2, ids[lo:hi]) and torch.equal(g2, gates[lo:hi])


@pytest.mark.parametrize("n,d,e,k", [(1, 64, 16, 1), (8, 5120, 16, 1), (64, 96, 128, 2), (1000, 80, 5, 3), (1024, 64, 9, 8),
                                     (1025, 64, 7, 2), (900, 64, 4000, 1), (3000, 72, 16, 1)])
def test_router_and_grouping_in_one_call(ops, n, d, e, k):
    """Few tokens: one block chooses and groups; many tokens, or tables too long for its shared memory: the separate
    kernels.  Either way the same as route, then align."""
    h, w = _rand(n, d, seed=1), _rand(e, d, scale=0.05, seed=2)
    ids, gates, logits = ops.moe_route(h, w, k, want_logits=True)
    ids2, gates2, logits2, grouping = ops.moe_route(h, w, k, want_logits=True, group=True)
    assert torch.equal(ids, ids2) and torch.equal(gates, gates2) and torch.equal(logits, logits2)
    want = ops.moe_align(ids, gates, e, extra_group=True)
    for a, b in zip(want, grouping):
        assert torch.equal(a, b)


def test_moe_route_lowest_index_wins_ties(ops):
    h = _rand(5, 64, seed=1)
    w = _rand(1, 64, seed=2).expand(6, 64).contiguous()  # every expert the same score
    ids, gates = ops.moe_route(h, w, 3)
    assert ids.tolist() == [[0, 1, 2]] * 5


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("n,d,f,e,k", [(50, 96, 40, 16, 1), (9, 80, 56, 3, 2), (130, 64, 24, 5, 1), (1, 64, 32, 4, 1)])
def test_moe_experts(ops, ref, dt, n, d, f, e, k):
    h = _rand(n, d, dt=dt, seed=1)
    wgu, wd = _rand(e, 2 * f, d, dt=dt, scale=0.2, seed=2), _rand(e, d, f, dt=dt, scale=0.2, seed=3)
    shared = _rand(n, d, dt=dt, seed=4)
    g = torch.Generator().manual_seed(5)
    ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
    if e > 3:
        ids[ids == 2] = 0  # an expert nobody chose
    gates = torch.rand(n, k, generator=g).to(DEV)
    lazy = ops.moe_experts(h, ids, gates, wgu, wd, shared)  # the pieces; summed by the kernel that uses them
    got = ops.materialize(lazy)
    want = ref.moe_experts(h, ids, gates, wgu, wd, shared)
    assert got.dtype == torch.float32 and lazy.shape == (n, d)
    _assert_close_to_scale(got, want, dt)
    _assert_close_to_scale(ops.materialize(ops.moe_experts(h, ids, gates, wgu, wd, None)),
                           ref.moe_experts(h, ids, gates, wgu, wd, None), dt)
    # residual add + norm reading the pieces = the same on the summed tensor
    x = _rand(n, d, seed=9)
    w = _rand(d, seed=10)
    x1, x2 = x.clone(), x.clone()
    h1, h32 = ops.add_rmsnorm(x1, lazy, w, 1e-5, dt, True)
    h2, h32b = ops.add_rmsnorm(x2, got, w, 1e-5, dt, True)
    assert torch.allclose(x1, x2, rtol=1e-6, atol=1e-6) and torch.allclose(h32, h32b, rtol=1e-5, atol=1e-6)
    x3 = x.clone()
    ops.add_residual(x3, lazy)
    assert torch.allclose(x3, x1, rtol=1e-6, atol=1e-6)
    idx = torch.tensor([n - 1, 0], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.gather_rows(lazy, idx), got[idx.long()])


_SHARED_CASES = [(1, 64, 32, 4, 1), (9, 96, 48, 3, 2), (16, 256, 64, 16, 1), (17, 64, 32, 4, 1), (50, 96, 48, 5, 1)]


# (the streaming layout exists for bfloat16 matrices of whole 16 x 32 tiles only)
@pytest.mark.parametrize("dt,tiled,n,d,f,e,k",
                         [(dt, False, *c) for dt in DT for c in _SHARED_CASES] +
                         [(torch.bfloat16, True, *c) for c in _SHARED_CASES if c[1] % 32 == 0 and c[2] % 32 == 0])
def test_moe_experts_with_the_shared_expert_given_by_its_matrices(ops, ref, dt, tiled, n, d, f, e, k):
    """Up to 16 tokens the shared expert's products go through the routed experts' launches as one more group
    (its matrices stay row-major beside experts in either layout); beyond, through the library.  The same sum."""
    from jax_llm_examples_amd.ops.layout import can_tile, tile_

    h = _rand(n, d, dt=dt, seed=1)
    wgu, wd = _rand(e, 2 * f, d, dt=dt, scale=0.2, seed=2), _rand(e, d, f, dt=dt, scale=0.2, seed=3)
    sgu, sd = _rand(2 * f, d, dt=dt, scale=0.2, seed=4), _rand(d, f, dt=dt, scale=0.2, seed=5)
    g = torch.Generator().manual_seed(5)
    ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
    gates = torch.rand(n, k, generator=g).to(DEV)
    want = ref.moe_experts(h, ids, gates, wgu, wd, shared_weights=(sgu, sd))
    if tiled:
        assert can_tile(wgu) and can_tile(wd)
        wgu, wd = wgu.clone(), wd.clone()
        tile_(wgu)
        tile_(wd)
    lazy = ops.moe_experts(h, ids, gates, wgu, wd, shared_weights=(sgu, sd), tiled=tiled)
    _assert_close_to_scale(ops.materialize(lazy), want, dt)
    # with the grouping that the router's own call makes (an extra group always), and with one made without
    for extra in (True, False):
        grouping = ops.moe_align(ids, gates, e, extra_group=extra)
        lazy = ops.moe_experts(h, ids, gates, wgu, wd, shared_weights=(sgu, sd), tiled=tiled, grouping=grouping)
        _assert_close_to_scale(ops.materialize(lazy), want, dt)


@pytest.mark.parametrize("n", [1, 8, 64, 2048])
def test_moe_experts_with_128_experts_most_of_them_empty_or_nearly(ops, ref, n):
    """128 experts at serving width (129 groups with the shared expert riding): one token leaves 127 experts
    empty, 2,048 tokens give each about 16 rows and some none (ten experts are never chosen here)."""
    from jax_llm_examples_amd.ops.layout import can_tile, tile_

    dt, d, f, e = torch.bfloat16, 5120, 512, 128
    h = _rand(n, d, dt=dt, seed=1)
    wgu, wd = _rand(e, 2 * f, d, dt=dt, scale=0.02, seed=2), _rand(e, d, f, dt=dt, scale=0.05, seed=3)
    sgu, sd = _rand(2 * f, d, dt=dt, scale=0.02, seed=4), _rand(d, f, dt=dt, scale=0.05, seed=5)
    g = torch.Generator().manual_seed(n)
    ids = (torch.randint(0, e - 10, (n, 1), generator=g) + 5).to(torch.int32).to(DEV)
    gates = torch.rand(n, 1, generator=g).to(DEV)
    want = ref.moe_experts(h, ids, gates, wgu, wd, shared_weights=(sgu, sd))
    assert can_tile(wgu) and can_tile(wd)
    tgu, td = wgu.clone(), wd.clone()
    tile_(tgu)
    tile_(td)
    for tiled, a, b in ((True, tgu, td), (False, wgu, wd)):
        for extra in (True, False):
            grouping = ops.moe_align(ids, gates, e, extra_group=extra)
            lazy = ops.moe_experts(h, ids, gates, a, b, shared_weights=(sgu, sd), tiled=tiled, grouping=grouping)
            _assert_close_to_scale(ops.materialize(lazy), want, dt)
    # the sum that the next norm reads piece by piece
    x = _rand(n, d, seed=7)
    lazy = ops.moe_experts(h, ids, gates, tgu, td, shared_weights=(sgu, sd), tiled=True)
    normed, _ = ops.add_rmsnorm(x.clone(), lazy, None, 1e-5, dt)
    ref_normed, _ = ref.add_rmsnorm(x.clone(), ops.materialize(lazy), None, 1e-5, dt)
    _assert_close_to_scale(normed, ref_normed, dt)


def test_moe_align_is_a_stable_grouping(ops):
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, 7, (300, 2), generator=g).to(torch.int32).to(DEV)
    gates = torch.rand(300, 2, generator=g).to(DEV)
    off, tok, gate, inv = ops.moe_align(ids, gates, 7)
    flat = ids.flatten().cpu()
    off, tok, gate, inv = off.cpu(), tok.cpu(), gate.cpu(), inv.cpu()
    assert off[0] == 0 and off[-1] == 600
    for e in range(7):
        rows = (flat == e).nonzero().squeeze(-1)
        assert off[e + 1] - off[e] == rows.numel()
        assert torch.equal(inv[rows], torch.arange(int(off[e]), int(off[e + 1]), dtype=torch.int32))  # in order
        assert torch.equal(tok[off[e]: off[e + 1]], (rows // 2).to(torch.int32))
    assert torch.equal(gate[inv.long()], gates.flatten().cpu())
    # one more group that holds every token once
    off2, tok2, gate2, inv2 = (t.cpu() for t in ops.moe_align(ids, gates, 7, extra_group=True))
    assert torch.equal(off2[:8], off) and off2[8] == 900 and torch.equal(inv2, inv)
    assert torch.equal(tok2[:600], tok) and torch.equal(tok2[600:], torch.arange(300, dtype=torch.int32))
    assert torch.equal(gate2[:600], gate) and torch.equal(gate2[600:], torch.ones(300))


@pytest.mark.parametrize("dt", DT)
def test_product_kernel_and_lm_head(ops, ref, dt):
    a, b = _rand(33, 52, dt=dt, seed=1), _rand(70, 52, dt=dt, seed=2)
    _assert_close_to_scale(ops.gemm(a, b), ref.linear(a, b), dt)
    gu = _rand(2 * 24, 52, dt=dt, seed=6)
    for rows in (33, 100):  # few rows (weight streaming in bfloat16) and many
        aa = _rand(rows, 52, dt=dt, seed=7)
        _assert_close_to_scale(ops.swiglu_linear(aa, gu), ref.swiglu_linear(aa, gu), dt)
        _assert_close_to_scale(ops.linear(aa, b), ref.linear(aa, b), dt)
    h, w = _rand(5, 80, dt=dt, seed=3), _rand(311, 80, dt=dt, seed=4)
    got = ops.lm_head(h, w)
    assert got.dtype == torch.float32 and got.shape == (5, 311)
    assert torch.allclose(got, ref.lm_head(h, w), rtol=2e-5, atol=2e-5)  # float32 accumulation and output
    _assert_close_to_scale(ops.linear(h, w), ref.linear(h, w), dt)


def test_float32_products_are_true_float32(ops):
    # a reduced-precision matrix mode (tf32/xf32: 10 mantissa bits) would lose the small term
    a = torch.tensor([[1.0, 2.0 ** -14]], device=DEV).repeat(4, 64)  # 128 columns
    b = torch.ones(8, 128, device=DEV)
    want = 64 * (1.0 + 2.0 ** -14)
    for out in (ops.linear(a, b), ops.lm_head(a, b), ops.gemm(a, b)):
        assert torch.allclose(out, torch.full_like(out, want), rtol=1e-7)


@pytest.mark.parametrize("rows", [1, 64, 2048])
@pytest.mark.parametrize("k", [5120, 8192, 16384])
def test_float32_products_are_true_float32_at_serving_sizes(ops, rows, k):
    """The shapes the dense projections really have (which algorithm a library picks depends on them), against
    a float64 product.  Rows of 1 + 2^-12, -1, 1 + 2^-12, -1, ... times ones: every partial sum over neighbouring
    terms is exact in float32 in whatever order it is taken, and the result is k / 2 * 2^-12; a mode that keeps
    10 mantissa bits of the operands gives 0.  And random operands against the float64 product."""
    nout = 384
    a = torch.tensor([[1.0 + 2.0 ** -12, -1.0]], device=DEV).repeat(rows, k // 2)
    b = torch.ones(nout, k, device=DEV)
    exact = k / 2 * 2.0 ** -12
    ar, br = _rand(rows, k, seed=11), _rand(nout, k, seed=12)
    want = (ar.double() @ br.double().t())
    scale = (ar.double().abs() @ br.double().abs().t())
    for name, fn in (("linear", ops.linear), ("lm_head", ops.lm_head), ("gemm", ops.gemm)):
        out = fn(a, b)
        assert float((out.double() - exact).abs().max()) <= 1e-6 * exact, name
        err = float(((fn(ar, br).double() - want).abs() / scale).max())
        assert err < 2e-6, f"{name}: {err:.3g} of the sum of the terms' sizes"


@pytest.mark.parametrize("n,d,f,e,k", [(1, 64, 32, 4, 1), (8, 5120, 96, 16, 1), (64, 260, 36, 128, 2), (100, 128, 64, 5, 1),
                                       (128, 512, 256, 16, 1), (50, 1028, 44, 3, 2), (129, 64, 16, 1, 1)])
def test_float32_grouped_product_on_the_float32_matrix_instructions(ops, n, d, f, e, k):
    """The weight-streaming float32 product (gemm_f32.hip) against float64: grouped, gathered, scaled, with and
    without the fused activation; sizes that leave partial tiles, chunks and groups without rows."""
    h = _rand(n, d, seed=1)
    wgu, wd = _rand(e, 2 * f, d, scale=0.1, seed=2), _rand(e, d, f, scale=0.1, seed=3)
    g = torch.Generator().manual_seed(n)
    ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
    if e > 2:
        ids[ids == 1] = 2  # a group without rows
    gates = torch.rand(n, k, generator=g).to(DEV)
    off, tok, gate, inv = ops.moe_align(ids, gates, e)
    act = ops.gemm_f32_skinny(h, wgu, offsets=off, a_rows=tok, scale=gate, swiglu=True)
    gu = ops.gemm_f32_skinny(h, wgu, offsets=off, a_rows=tok, scale=gate)
    sorted_ids = ids.flatten()[torch.argsort(inv.long())].long()
    x64 = h.double()[tok.long()] * gate.double()[:, None]
    want_gu = torch.einsum("nk,nok->no", x64, wgu.double()[sorted_ids])
    want_act = torch.nn.functional.silu(want_gu[:, :f]) * want_gu[:, f:]
    assert float((gu.double() - want_gu).abs().max() / want_gu.abs().max()) <= 3e-6
    assert float((act.double() - want_act).abs().max() / want_act.abs().max()) <= 3e-6
    out = ops.gemm_f32_skinny(act, wd, offsets=off)
    want = torch.einsum("nk,nok->no", act.double(), wd.double()[sorted_ids])
    assert float((out.double() - want).abs().max() / want.abs().max()) <= 3e-6
    # one group without offsets, and the result of a row does not depend on what else is in the launch
    dense = ops.gemm_f32_skinny(h, wgu[0])
    assert float((dense.double() - h.double() @ wgu[0].double().t()).abs().max() / dense.abs().max()) <= 3e-6
    assert torch.equal(ops.gemm_f32_skinny(h[:1].contiguous(), wgu[0]), dense[:1])
    with pytest.raises(Exception, match="multiple of 4"):
        ops.gemm_f32_skinny(h[:, : d - 2].contiguous(), wgu[:, :, : d - 2].contiguous())


@pytest.mark.parametrize("n,d,f,e,k", [(1, 64, 64, 4, 1), (50, 128, 64, 4, 1), (300, 192, 128, 3, 2), (700, 64, 192, 5, 1),
                                       (450, 320, 64, 2, 1), (2100, 5120, 128, 16, 1), (200, 1088, 448, 128, 2)])
def test_float32_grouped_product_for_many_rows_on_the_float32_matrix_instructions(ops, n, d, f, e, k):
    """The float32 product whose wavefronts hold up to 192 rows of a group (gemm_f32.hip) against float64: grouped,
    gathered, scaled, with and without the fused activation; groups of more than 192 rows (several passes), of a
    few rows and of none, rows that fill no tile."""
    h = _rand(n, d, seed=1)
    wgu, wd = _rand(e, 2 * f, d, scale=0.1, seed=2), _rand(e, d, f, scale=0.1, seed=3)
    g = torch.Generator().manual_seed(n)
    ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
    if e > 2:
        ids[ids == 1] = 2  # a group without rows, and one with twice its share
    gates = torch.rand(n, k, generator=g).to(DEV)
    off, tok, gate, inv = ops.moe_align(ids, gates, e)
    act = ops.gemm_f32_stream(h, wgu, offsets=off, a_rows=tok, scale=gate, swiglu=True)
    gu = ops.gemm_f32_stream(h, wgu, offsets=off, a_rows=tok, scale=gate)
    sorted_ids = ids.flatten()[torch.argsort(inv.long())].long()
    x64 = h.double()[tok.long()] * gate.double()[:, None]
    want_gu = torch.empty(tok.numel(), 2 * f, dtype=torch.float64, device=DEV)
    for j in range(e):
        rows = sorted_ids == j
        want_gu[rows] = x64[rows] @ wgu[j].double().t()
    want_act = torch.nn.functional.silu(want_gu[:, :f]) * want_gu[:, f:]
    assert float((gu.double() - want_gu).abs().max() / want_gu.abs().max()) <= 3e-6
    assert float((act.double() - want_act).abs().max() / want_act.abs().max()) <= 3e-6
    out = ops.gemm_f32_stream(act, wd, offsets=off)
    want = torch.empty(tok.numel(), d, dtype=torch.float64, device=DEV)
    for j in range(e):
        rows = sorted_ids == j
        want[rows] = act.double()[rows] @ wd[j].double().t()
    assert float((out.double() - want).abs().max() / want.abs().max()) <= 3e-6
    # one group without offsets, and the result of a row does not depend on what else is in the launch
    # (measured against the sum of the terms' sizes, as for the dense projections above: the sums over 5,120 terms
    # are formed one stage after the other)
    dense = ops.gemm_f32_stream(h, wgu[0])
    terms = h.double().abs() @ wgu[0].double().abs().t()
    assert float(((dense.double() - h.double() @ wgu[0].double().t()).abs() / terms).max()) < 2e-6
    assert torch.equal(ops.gemm_f32_stream(h[:1].contiguous(), wgu[0]), dense[:1])
    with pytest.raises(Exception, match="multiple of 64"):
        ops.gemm_f32_stream(h[:, : d - 32].contiguous(), wgu[:, :, : d - 32].contiguous())
    # through the experts' entry: more rows than the few-rows kernel takes
    if n * k > ops.F32_SKINNY_ROWS:
        calls = []
        inner = ops._call
        ops._call = lambda name, *a: (calls.append(name), inner(name, *a))[1]
        try:
            got = ops.materialize(ops.moe_experts(h, ids, gates, wgu, wd, None))
        finally:
            ops._call = inner
        assert calls.count("jle_gemm_f32_stream") == 2, calls
        want_sum = torch.zeros(n, d, dtype=torch.float64, device=DEV)
        want_sum.index_add_(0, tok.long(), want)
        assert float((got.double() - want_sum).abs().max() / want_sum.abs().max()) <= 3e-6


def test_sampling(ops, ref):
    g = torch.Generator().manual_seed(0)
    V = 1000
    logits = torch.randn(6, V, generator=g).to(DEV)
    logits[0, 17] = logits[0, 400] = 9.0  # two equal maxima: the lower id
    z = torch.zeros(6, dtype=torch.int32, device=DEV)
    greedy = ops.sample(logits, torch.zeros(6, device=DEV), z, z, z)
    assert greedy.tolist() == torch.argmax(logits, -1).tolist() and greedy[0] == 17
    temp = torch.tensor([0.0, 0.7, 1.0, 1.3, 1.0, 1.0], device=DEV)
    topk = torch.tensor([0, 0, 5, 16, 1, 0], dtype=torch.int32, device=DEV)
    seeds = torch.tensor([1, 2, 3, 4, 5, 6], dtype=torch.int32, device=DEV)
    for c in range(4):
        ctr = torch.full((6,), c, dtype=torch.int32, device=DEV)
        got = ops.sample(logits, temp, topk, seeds, ctr)
        want = ref.sample(logits.cpu(), temp.cpu(), topk.cpu(), seeds.cpu(), ctr.cpu())
        assert got.tolist() == want.tolist()
        assert got[4] == torch.argmax(logits[4])  # top_k = 1 is greedy
        assert int(got[2]) in torch.topk(logits[2], 5).indices.tolist()
    # a request's draw does not depend on what else is in the batch
    alone = ops.sample(logits[3:4].contiguous(), temp[3:4].contiguous(), topk[3:4].contiguous(),
                       seeds[3:4].contiguous(), torch.tensor([2], dtype=torch.int32, device=DEV))
    ctr = torch.full((6,), 2, dtype=torch.int32, device=DEV)
    assert alone[0] == ops.sample(logits, temp, topk, seeds, ctr)[3]


def test_sampling_frequencies_follow_softmax(ops):
    p = torch.tensor([0.5, 0.25, 0.15, 0.07, 0.03])
    n = 4000
    logits = torch.log(p)[None].repeat(n, 1).to(DEV) * 2.0  # temperature 2 undoes the factor
    out = ops.sample(logits, torch.full((n,), 2.0, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV),
                     torch.arange(n, dtype=torch.int32, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV))
    freq = torch.bincount(out.cpu().long(), minlength=5).float() / n
    sigma = torch.sqrt(p * (1 - p) / n)
    assert ((freq - p).abs() < 4 * sigma).all(), (freq, p)


@pytest.mark.parametrize("m,nout,k", [(1, 64, 64), (8, 70, 104), (16, 33, 32), (17, 96, 40), (40, 500, 264),
                                       (64, 130, 5120), (5, 1000, 8192), (3, 80, 1096)])
@pytest.mark.parametrize("out_f32", [False, True])
def test_weight_streaming_product(ops, ref, m, nout, k, out_f32):
    a, b = _rand(m, k, dt=torch.bfloat16, seed=1), _rand(nout, k, dt=torch.bfloat16, scale=0.1, seed=2)
    got = ops.gemm_skinny(a, b, out_f32=out_f32)
    want = a.float() @ b.float().t()
    assert got.dtype == (torch.float32 if out_f32 else torch.bfloat16)
    err = float((got.float() - want).abs().max() / want.abs().max())
    assert err <= (2e-5 if out_f32 else 5e-3), err  # float32 out: only the order of the sum differs


@pytest.mark.parametrize("m", [1, 8, 16])
@pytest.mark.parametrize("nout,k", [(5120, 320), (5120, 8192), (1024, 264), (9216, 5120), (2048, 512)])
def test_weight_streaming_product_with_row_tiles_cut_along_k(ops, m, nout, k):
    """Row tiles that do not fill a round of the compute units are cut along K, each slice a block of its own,
    and the slices' sums are added by the tile's last block in the slices' order: the same bits every time, in
    both layouts, and the tickets are back at zero."""
    from jax_llm_examples_amd.ops.layout import can_tile, tile_
    tiles = -(-nout // 16)
    cut, slices = ops._k_slices(tiles)
    assert cut > 0 and (cut * slices) % ops._compute_units == 0, "sizes chosen so that tiles are cut"
    a, b = _rand(m, k, dt=torch.bfloat16, seed=1), _rand(nout, k, dt=torch.bfloat16, scale=0.1, seed=2)
    want = a.float() @ b.float().t()
    got = ops.gemm_skinny(a, b, out_f32=True)
    assert float((got - want).abs().max() / want.abs().max()) <= 2e-5
    whole = ops.gemm_skinny(a, b, out_f32=True, balance=False)  # (sums in another order: other blocks, other bits)
    assert float((whole - want).abs().max() / want.abs().max()) <= 2e-5
    for _ in range(3):
        assert torch.equal(ops.gemm_skinny(a, b, out_f32=True), got)
    if can_tile(b):
        bt = b.clone()
        tile_(bt)
        assert torch.equal(ops.gemm_skinny(a, bt, out_f32=True, tiled=True), got)
    assert int(ops._slice_tickets.abs().sum()) == 0


@pytest.mark.parametrize("n,e,nout,k", [(1, 16, 5120, 512), (2, 128, 5120, 256), (8, 16, 5120, 8192), (7, 128, 320, 64),
                                        (16, 40, 2048, 128)])
def test_weight_streaming_product_over_group_slots(ops, n, e, nout, k):
    """A grouped product of few rows is launched over as many group slots as it has rows (slot j: the j-th group
    that has rows), with a last group whose matrix is a tensor of its own: the same result as over every group."""
    dt = torch.bfloat16
    g = torch.Generator().manual_seed(n)
    ids = torch.randint(0, e, (n, 1), generator=g).to(torch.int32).to(DEV)
    gates = torch.rand(n, 1, generator=g).to(DEV)
    off, tok, gate, inv = ops.moe_align(ids, gates, e, extra_group=True)
    x = _rand(2 * n, k, dt=dt, seed=1)  # (rows already grouped: the second product of an expert layer)
    w, w_last = _rand(e, nout, k, dt=dt, scale=0.1, seed=2), _rand(nout, k, dt=dt, scale=0.1, seed=3)
    got = ops.gemm_skinny(x, w, offsets=off, b_last=w_last, out_f32=True)
    every = ops.gemm_skinny(x, w, offsets=off, b_last=w_last, out_f32=True, balance=False)
    sorted_ids = ids.flatten()[tok[:n].long()].long()
    want = torch.cat([torch.einsum("nk,nok->no", x[:n].float(), w[sorted_ids].float()),
                      x[n:].float() @ w_last.float().t()])
    assert float((got - want).abs().max() / want.abs().max()) <= 2e-5
    assert float((every - want).abs().max() / want.abs().max()) <= 2e-5
    # (tiles are cut only in launches of one or two group slots; with no tile cut the same blocks form the same sums)
    if ops._k_slices(-(-nout // 16))[0] == 0 or 2 * n > ops.CUT_SLOTS:
        assert torch.equal(got, every)
    # gathered rows, scaled, with the fused activation (the first product of an expert layer)
    h = _rand(n, k, dt=dt, seed=4)
    wgu, wgu_last = _rand(e, 2 * 64, k, dt=dt, scale=0.1, seed=5), _rand(2 * 64, k, dt=dt, scale=0.1, seed=6)
    a1 = ops.gemm_skinny(h, wgu, offsets=off, a_rows=tok, scale=gate, swiglu=True, b_last=wgu_last, rows=2 * n)
    a2 = ops.gemm_skinny(h, wgu, offsets=off, a_rows=tok, scale=gate, swiglu=True, b_last=wgu_last, rows=2 * n,
                         balance=False)
    assert torch.equal(a1, a2)
    assert int(ops._slice_tickets.abs().sum()) == 0


@pytest.mark.parametrize("n,d,f,e,k", [(8, 128, 48, 16, 1), (64, 5120, 64, 16, 1), (20, 264, 40, 3, 2), (3, 64, 24, 128, 1)])
def test_weight_streaming_product_grouped_with_swiglu(ops, ref, n, d, f, e, k):
    dt = torch.bfloat16
    h = _rand(n, d, dt=dt, seed=1)
    wgu = _rand(e, 2 * f, d, dt=dt, scale=0.1, seed=2)
    g = torch.Generator().manual_seed(5)
    ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
    if n == 64:
        ids[:40] = 3  # one expert with more rows than one tile of 16
    gates = torch.rand(n, k, generator=g).to(DEV)
    off, tok, gate, inv = ops.moe_align(ids, gates, e)
    act = ops.gemm_skinny(h, wgu, offsets=off, a_rows=tok, scale=gate, swiglu=True)
    gu = ops.gemm(h, wgu, offsets=off, a_rows=tok, scale=gate, out_f32=True)  # the general kernel, float32 result
    want = torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]
    assert act.shape == (n * k, f)
    assert float((act.float() - want).abs().max() / want.abs().max()) <= 5e-3
    plain = ops.gemm_skinny(h, wgu, offsets=off, a_rows=tok, scale=gate, out_f32=True)
    assert float((plain - gu).abs().max() / gu.abs().max()) <= 2e-5


@pytest.mark.parametrize("n,d,f,e,k", [(300, 128, 48, 16, 1), (700, 264, 72, 3, 2), (2048, 512, 256, 16, 1),
                                       (150, 64, 40, 128, 1)])
def test_grouped_product_for_many_rows(ops, ref, n, d, f, e, k):
    dt = torch.bfloat16
    h = _rand(n, d, dt=dt, seed=1)
    wgu = _rand(e, 2 * f, d, dt=dt, scale=0.1, seed=2)
    wd = _rand(e, d, f, dt=dt, scale=0.1, seed=3)
    g = torch.Generator().manual_seed(5)
    ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
    if n == 300:
        ids[:200] = 3  # one expert with more rows than one block, others with none
    gates = torch.rand(n, k, generator=g).to(DEV)
    off, tok, gate, inv = ops.moe_align(ids, gates, e)
    act = ops.gemm_grouped(h, wgu, offsets=off, a_rows=tok, scale=gate, swiglu=True)
    gu = ops.gemm(h, wgu, offsets=off, a_rows=tok, scale=gate, out_f32=True)  # the general kernel, float32 result
    want = torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]
    assert act.shape == (n * k, f)
    assert float((act.float() - want).abs().max() / want.abs().max()) <= 5e-3
    plain = ops.gemm_grouped(h, wgu, offsets=off, a_rows=tok, scale=gate, out_f32=True)
    assert float((plain - gu).abs().max() / gu.abs().max()) <= 2e-5
    down = ops.gemm_grouped(act, wd, offsets=off)
    want_d = ops.gemm(act, wd, offsets=off, out_f32=True)
    assert float((down.float() - want_d).abs().max() / want_d.abs().max()) <= 5e-3
    # the whole expert layer at this size takes the same path
    _assert_close_to_scale(ops.materialize(ops.moe_experts(h, ids, gates, wgu, wd, None)),
                           ref.moe_experts(h, ids, gates, wgu, wd, None), dt)
    dense = ops.gemm_grouped(h, wgu[0], out_f32=True)  # one group, no offsets
    assert float((dense - h.float() @ wgu[0].float().t()).abs().max() / dense.abs().max()) <= 2e-5
    head = ops.lm_head(h[:100, :], _rand(311, d, dt=dt, seed=7))
    assert head.dtype == torch.float32 and head.shape == (100, 311)


@pytest.mark.parametrize("n,d,f,e,k", [(300, 256, 32, 16, 1), (700, 768, 96, 3, 2), (2048, 512, 256, 16, 1),
                                       (150, 256, 48, 128, 1), (900, 256, 80, 2, 1)])
def test_weight_streaming_grouped_product(ops, ref, n, d, f, e, k):
    """Groups without rows, with a few, with more than one pass of 192; an odd number of weight tiles."""
    from jax_llm_examples_amd.ops.layout import tile_
    dt = torch.bfloat16
    h = _rand(n, d, dt=dt, seed=1)
    wgu = _rand(e, 2 * f, d, dt=dt, scale=0.1, seed=2)
    wd = _rand(e, d, f, dt=dt, scale=0.1, seed=3)
    g = torch.Generator().manual_seed(5)
    ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
    if n == 300:
        ids[:270] = 3  # one expert with more rows than one pass, others with none
    gates = torch.rand(n, k, generator=g).to(DEV)
    off, tok, gate, inv = ops.moe_align(ids, gates, e)
    wgu_t = wgu.clone()
    tile_(wgu_t)
    gu = ops.gemm(h, wgu, offsets=off, a_rows=tok, scale=gate, out_f32=True)  # the general kernel, float32 result
    plain = ops.gemm_stream(h, wgu_t, offsets=off, a_rows=tok, scale=gate, out_f32=True)
    assert float((plain - gu).abs().max() / gu.abs().max()) <= 2e-5
    if f % 16 == 0:
        act = ops.gemm_stream(h, wgu_t, offsets=off, a_rows=tok, scale=gate, swiglu=True)
        want = torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]
        assert act.shape == (n * k, f)
        assert float((act.float() - want).abs().max() / want.abs().max()) <= 5e-3
    else:
        with pytest.raises(Exception, match="refuses|needs"):
            ops.gemm_stream(h, wgu_t, offsets=off, a_rows=tok, scale=gate, swiglu=True)
        act = ops.gemm_grouped(h, wgu, offsets=off, a_rows=tok, scale=gate, swiglu=True)
    if f % 256 == 0:
        wd_t = wd.clone()
        tile_(wd_t)
        down = ops.gemm_stream(act, wd_t, offsets=off)
        want_d = ops.gemm(act, wd, offsets=off, out_f32=True)
        assert float((down.float() - want_d).abs().max() / want_d.abs().max()) <= 5e-3
    dense = ops.gemm_stream(h, wgu_t[0], out_f32=True)  # one group, no offsets
    assert float((dense - h.float() @ wgu[0].float().t()).abs().max() / dense.abs().max()) <= 2e-5
    with pytest.raises(Exception, match="refuses|needs"):
        ops.gemm_stream(h[:, :d - 128].contiguous(), wgu_t[:, :, :d - 128].contiguous())


def test_streaming_layout_gives_the_same_results_bit_for_bit(ops):
    from jax_llm_examples_amd.ops.layout import can_tile, tile_, untiled
    dt = torch.bfloat16
    w = _rand(3, 96, 160, dt=dt, seed=1)
    wt = w.clone()
    assert can_tile(w) and not can_tile(_rand(3, 90, 160, dt=dt)) and not can_tile(w.float())
    tile_(wt)
    assert not torch.equal(wt, w) and torch.equal(untiled(wt), w)
    first_tile = wt[1].flatten()[:512].reshape(4, 16, 8)  # the first kilobyte: rows 0..15, k 0..31 as [g][r][8]
    assert torch.equal(first_tile[2, 5], w[1, 5, 16:24])
    second = wt[1].flatten()[512:1024].reshape(4, 16, 8)  # the next tile goes on along K
    assert torch.equal(second[0, 3], w[1, 3, 32:40])
    for n, d, f, e, k in [(8, 128, 48, 16, 1), (50, 160, 96, 5, 2), (400, 256, 64, 4, 1)]:
        h = _rand(n, d, dt=dt, seed=1)
        wgu, wd = _rand(e, 2 * f, d, dt=dt, scale=0.1, seed=2), _rand(e, d, f * 1, dt=dt, scale=0.1, seed=3)
        if f % 32:
            continue
        g = torch.Generator().manual_seed(5)
        ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(DEV)
        gates = torch.rand(n, k, generator=g).to(DEV)
        wgu_t, wd_t = wgu.clone(), wd.clone()
        tile_(wgu_t), tile_(wd_t)
        a = ops.materialize(ops.moe_experts(h, ids, gates, wgu, wd, None))
        b = ops.materialize(ops.moe_experts(h, ids, gates, wgu_t, wd_t, None, tiled=True))
        assert torch.equal(a, b)
    for m in (3, 40, 200):
        h, w2 = _rand(m, 160, dt=dt, seed=4), _rand(17 * 16, 160, dt=dt, seed=5)  # an odd number of row tiles
        w2t = w2.clone()
        tile_(w2t)
        assert torch.equal(ops.lm_head(h, w2), ops.lm_head(h, w2t, tiled=True))
