"""GPU parity tests of the Llama decode operators (autort.ops.rmsnorm_*, rotary_*,
rotate_*, attention_*) against the CPU oracle.  fp32: 1e-5, fp16: rtol/atol 1e-2."""
import math

import numpy as np
import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures('oracle_built')]

FP32_TOL = dict(rtol=1e-5, atol=1e-5)
FP16_TOL = dict(rtol=1e-2, atol=1e-2)


@pytest.fixture(scope='module')
def autort():
    import autort as mod
    return mod


def note(msg):
    print(f'[case] {msg}', flush=True)


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize('n', [64, 4096, 11008, 1000])
def test_rmsnorm_f32_like_the_sample(autort, n):
    """samples/05_llama2_7b_int4.py:128-131: torch computes vsum, the op normalises."""
    from oracle import hot_ops
    note(f'rmsnorm_f32 n={n}')
    dev = autort.device()
    x = torch.randn(1, n, generator=gen(n))
    w = 1 + 0.1 * torch.randn(n, generator=gen(n + 1))
    xd = x.to(dev).float()
    vsum = (xd * xd).sum().view(1)
    out = autort.ops.rmsnorm_f32(xd.view(-1), vsum, w.to(dev).float(), extra=[1.0 / int(xd.numel())])
    want = hot_ops.rmsnorm(x.numpy(), vsum.cpu().numpy(), w.numpy(), 1.0 / n)
    assert out.dtype == torch.float32 and out.shape == (n,)
    assert np.allclose(out.cpu().numpy(), want, **FP32_TOL)
    # fused sum of squares (vsum=None) agrees
    out2 = autort.ops.rmsnorm_f32(xd.view(-1), None, w.to(dev).float(), extra=[1.0 / n])
    assert np.allclose(out2.cpu().numpy(), hot_ops.rmsnorm(x.numpy(), None, w.numpy()), **FP32_TOL)


def test_rmsnorm_f16_variants(autort):
    from oracle import hot_ops
    note('rmsnorm_f16: fp32 x + fp16 w (sample 04), fp16 x + fp16 w')
    dev = autort.device()
    n = 4096
    x = torch.randn(n, generator=gen(1))
    w = (1 + 0.1 * torch.randn(n, generator=gen(2))).half()
    xd = x.to(dev)
    vsum = (xd * xd).sum().view(1)
    out = autort.ops.rmsnorm_f16(xd, vsum, w.to(dev), extra=[1.0 / n])
    assert out.dtype == torch.float16
    want = hot_ops.rmsnorm(x.numpy(), vsum.cpu().numpy(), w.numpy(), 1.0 / n, out_dtype=np.float16)
    assert np.allclose(out.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)
    xh = x.half()
    out = autort.ops.rmsnorm_f16(xh.to(dev), None, w.to(dev))
    want = hot_ops.rmsnorm(xh.numpy(), None, w.numpy(), out_dtype=np.float16)
    assert np.allclose(out.cpu().numpy().astype(np.float32), want.astype(np.float32), **FP16_TOL)


@pytest.mark.parametrize('dtype,pos', [(torch.float32, 0), (torch.float32, 5), (torch.float32, 383), (torch.float16, 77)])
def test_rotary_rotate_half(autort, dtype, pos):
    from oracle import hot_ops
    note(f'rotary {dtype} pos={pos}')
    dev = autort.device()
    H, D = 32, 128
    x = torch.randn(H * D, generator=gen(pos)).to(dtype)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D)).to(dtype))
    inv_freq = torch.cat([inv_freq, inv_freq]).view(D)
    op = autort.ops.rotary_f32 if dtype == torch.float32 else autort.ops.rotary_f16
    out = torch.empty(H, D, dtype=dtype, device=dev)
    r = op(x.to(dev).view(H, 2, -1), inv_freq.to(dev), out, extra=[pos])
    assert r.data_ptr() == out.data_ptr()
    want = hot_ops.rotary(x.numpy().reshape(H, 2, D // 2), inv_freq.numpy(), pos)
    tol = FP32_TOL if dtype == torch.float32 else FP16_TOL
    # fp32 sin/cos of angles up to 383 rad differ by a few ulp of the angle between libraries
    tol = dict(rtol=tol['rtol'], atol=max(tol['atol'], 1e-4 if pos > 100 else tol['atol']))
    assert np.allclose(out.cpu().numpy().astype(np.float32), want.astype(np.float32), **tol)
    # position read on the device gives the same bits
    pos_t = torch.tensor([pos], dtype=torch.int32, device=dev)
    out2 = op(x.to(dev).view(H, 2, -1), inv_freq.to(dev), torch.empty_like(out), extra=[pos_t])
    assert torch.equal(out, out2)


def test_rotate_interleaved(autort):
    from oracle import hot_ops
    note('rotate_f32 (interleaved pairs)')
    dev = autort.device()
    dim, head = 768, 64
    coef = (1 / torch.pow(1e4, torch.arange(0, dim, 2, dtype=torch.int64) % head / head)).view(1, -1).float()
    data = torch.randn(dim, generator=gen(3))
    out = torch.empty(dim, device=dev)
    autort.ops.rotate_f32(coef.to(dev), data.to(dev).view(-1), out.view(-1), extra=[9])
    assert np.allclose(out.cpu().numpy(), hot_ops.rotate(coef.numpy(), data.numpy(), 9), **FP32_TOL)


@pytest.mark.parametrize('dtype,S', [(torch.float32, 1), (torch.float32, 31), (torch.float32, 130), (torch.float16, 7), (torch.float16, 384)])
def test_attention_on_cache_views(autort, dtype, S):
    """k, v are narrow() views of a larger cache, as in samples/05_llama2_7b_int4.py:161-165."""
    from oracle import hot_ops
    note(f'attention {dtype} S={S}')
    dev = autort.device()
    H, D, seq_len = 32, 128, 400
    g = gen(S)
    key_cache = torch.randn(seq_len, H * D, generator=g).to(dtype).to(dev)
    val_cache = torch.randn(seq_len, H * D, generator=g).to(dtype).to(dev)
    q = torch.randn(H, D, generator=g).to(dtype).to(dev)
    att_f = torch.tensor([1 / math.sqrt(D)], dtype=torch.float32, device=dev)
    b_sk = key_cache.view(seq_len, H, D).narrow(0, 0, S)
    b_sv = val_cache.view(seq_len, H, D).narrow(0, 0, S)
    op = autort.ops.attention_f32 if dtype == torch.float32 else autort.ops.attention_f16
    out = op(q, b_sk, b_sv, att_f)
    want = hot_ops.attention(q.cpu().numpy(), b_sk.cpu().numpy(), b_sv.cpu().numpy(), float(att_f[0]))
    tol = FP32_TOL if dtype == torch.float32 else FP16_TOL
    assert out.shape == (H, D) and out.dtype == dtype
    assert np.allclose(out.cpu().numpy().astype(np.float32), want.astype(np.float32), **tol)
    # length taken from a device-side position
    pos_t = torch.tensor([S - 1], dtype=torch.int32, device=dev)
    out2 = op(q, key_cache.view(seq_len, H, D), val_cache.view(seq_len, H, D), att_f, extra=[pos_t])
    assert torch.equal(out, out2)


def test_greedy_next_matches_torch():
    """pos += 1; token = prompt[pos] while the prompt lasts, else argmax(logits) (first maximum); x = embed[token]."""
    import autort
    dev = autort.device()
    g = torch.Generator().manual_seed(4)
    V, D = 32000, 4096
    embed = (torch.randn(V, D, generator=g) * 0.02).half().to(dev)
    prompt = torch.randint(0, V, (5,), generator=g, dtype=torch.int32).to(dev)
    x = torch.zeros(D, dtype=torch.float16, device=dev)
    for case in range(6):
        note(f'greedy_next case {case}')
        logits = torch.randn(V, generator=g).half()
        if case == 1:                      # ties: the first maximum wins
            logits[[777, 20000, 31999]] = logits.max() + 1
        if case == 2:
            logits[V - 1] = 100.0          # last element
        if case == 3:
            logits[0] = 100.0              # first element
        logits = logits.to(dev)
        for start_pos, use_prompt in ((0, True), (3, True), (4, True), (9, True), (7, False)):
            token = torch.full((1,), -1, dtype=torch.int32, device=dev)
            pos = torch.full((1,), start_pos, dtype=torch.int32, device=dev)
            autort.ops.greedy_next_f16(logits, prompt if use_prompt else None, token, pos, embed, x)
            torch.cuda.synchronize()
            new_pos = start_pos + 1
            want = int(prompt[new_pos]) if (use_prompt and new_pos < prompt.numel()) else int(torch.argmax(logits.float().cpu()))
            if case == 1 and not (use_prompt and new_pos < prompt.numel()):
                want = 777
            assert int(pos) == new_pos and int(token) == want, (case, start_pos, use_prompt, int(token), want)
            assert torch.equal(x, embed[want])


@pytest.mark.parametrize('parts', [2, 4, 8])
@pytest.mark.parametrize('pos', [0, 1, 5, 130, 383])
def test_split_attention_merged_by_the_projection(parts, pos):
    """attention_rope_split_f16 + gemv_w4a16_attn against attention_rope_f16 + gemv_w4a16_fused (same caches, same
    token): the cache rows written must be identical, the projected outputs equal up to fp32 reassociation."""
    import autort
    from antares_amd import workloads
    dev = autort.device()
    H, D, S = 32, 128, 384
    g = torch.Generator().manual_seed(100 * parts + pos)
    note(f'split attention parts={parts} pos={pos}')
    qkv = torch.randn(3 * H * D, generator=g).half().to(dev)
    inv = (1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))).half()
    inv_freq = torch.cat([inv, inv]).to(dev)
    kc = (torch.randn(S, H * D, generator=g) * 0.5).half().to(dev)
    vc = torch.randn(S, H * D, generator=g).half().to(dev)
    att_f = torch.tensor([1 / math.sqrt(D)], dtype=torch.float32, device=dev)
    pos_t = torch.tensor([pos], dtype=torch.int32, device=dev)
    p = workloads.w4_problem(7, 1, H * D, 4096)
    qw, sc, qz = (p[k].to(dev) for k in ('qweight', 'scales', 'qzeros'))
    res = torch.randn(4096, generator=g).half().to(dev)
    # reference path: one block per head, then the fused projection
    kc1, vc1 = kc.clone(), vc.clone()
    att = torch.empty(H, D, dtype=torch.float16, device=dev)
    autort.ops.attention_rope_f16(qkv, inv_freq, kc1, vc1, att_f, att, extra=[pos_t])
    y1 = torch.empty(4096, dtype=torch.float16, device=dev)
    autort.ops.gemv_w4a16_fused(att.view(-1), qw, sc, qz, y1, residual=res)
    # split path
    kc2, vc2 = kc.clone(), vc.clone()
    partial = torch.full((H, parts, 132), float('nan'), dtype=torch.float32, device=dev)
    autort.ops.attention_rope_split_f16(qkv, inv_freq, kc2, vc2, att_f, partial, extra=[pos_t])
    y2 = torch.empty(4096, dtype=torch.float16, device=dev)
    autort.ops.gemv_w4a16_attn(partial, qw, sc, qz, y2, residual=res)
    torch.cuda.synchronize()
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    # merging the records by hand reproduces the unsplit attention output
    acc, mx, sm = partial[:, :, :128].double(), partial[:, :, 128].double(), partial[:, :, 129].double()
    wgt = torch.exp(mx - mx.max(dim=1, keepdim=True).values)
    wgt[torch.isinf(mx)] = 0
    merged = (acc * wgt[:, :, None]).sum(1) / (sm * wgt).sum(1)[:, None]
    assert torch.allclose(merged.float(), att.float(), rtol=2e-3, atol=2e-3)
    assert torch.allclose(y2.float(), y1.float(), rtol=1e-2, atol=1e-2)


def test_position_past_the_cache_touches_nothing(autort):
    """A position read on the device that lies past the last cache row (a recorded graph replayed once too often)
    must not run off the allocation: the cache-writing operators write nothing, the attention returns NaN."""
    note('device-side position == rows of the cache')
    dev = autort.device()
    H, D, ROWS = 4, 128, 6
    g = torch.Generator().manual_seed(3)
    backing_k = torch.randn(ROWS + 2, H * D, generator=g).half().to(dev)     # two guard rows behind the cache
    backing_v = torch.randn(ROWS + 2, H * D, generator=g).half().to(dev)
    key_cache, val_cache = backing_k[:ROWS], backing_v[:ROWS]
    before_k, before_v = backing_k.clone(), backing_v.clone()
    qkv = torch.randn(3 * H * D, generator=g).half().to(dev)
    inv = torch.rand(D, generator=g).half().to(dev)
    att_f = torch.tensor([0.1], dtype=torch.float32, device=dev)
    pos = torch.tensor([ROWS], dtype=torch.int32, device=dev)

    out = torch.zeros(H, D, dtype=torch.float16, device=dev)
    autort.ops.attention_rope_f16(qkv, inv, key_cache, val_cache, att_f, out, extra=[pos])
    assert torch.isnan(out).all()
    partial = torch.zeros(H, 4, 132, dtype=torch.float32, device=dev)
    autort.ops.attention_rope_split_f16(qkv, inv, key_cache, val_cache, att_f, partial, extra=[pos])
    assert torch.isnan(partial[:, :, :128]).all() and torch.isnan(partial[:, :, 129]).all()
    q_out = torch.zeros(H, D, dtype=torch.float16, device=dev)
    autort.ops.rope_qkv_store_f16(qkv, inv, q_out, key_cache, val_cache, extra=[pos])
    autort.ops.rotary_f16(qkv[:H * D].view(H, 2, -1), inv, key_cache, extra=[pos])
    out2 = torch.zeros(H, D, dtype=torch.float16, device=dev)
    autort.ops.attention_f16(q_out, key_cache.view(ROWS, H, D), val_cache.view(ROWS, H, D), att_f, out2, extra=[pos])
    assert torch.isnan(out2).all()
    torch.cuda.synchronize()
    assert torch.equal(backing_k, before_k) and torch.equal(backing_v, before_v)
    # the last valid position still works
    pos.fill_(ROWS - 1)
    autort.ops.attention_rope_f16(qkv, inv, key_cache, val_cache, att_f, out, extra=[pos])
    assert torch.isfinite(out).all()
    assert torch.equal(backing_k[ROWS:], before_k[ROWS:]) and torch.equal(backing_v[ROWS:], before_v[ROWS:])


@pytest.mark.usefixtures('oracle_built')
@pytest.mark.parametrize('parts', [1, 4, 8])
@pytest.mark.parametrize('pos', [0, 31, 130, 255, 256, 257, 383])
def test_fused_decode_attention_against_the_oracle(parts, pos):
    """The kernels the decode step runs - attention_rope_f16 (parts == 1) and attention_rope_split_f16 merged by
    gemv_w4a16_attn - against the oracle's rotary + attention (+ int4 projection) at the full head count, at
    positions on both sides of every 256-position round of the kernel, including the cache rows they write."""
    import autort
    from antares_amd import workloads
    from oracle import hot_ops
    dev = autort.device()
    H, D, S = 32, 128, 384
    g = torch.Generator().manual_seed(1000 * parts + pos)
    note(f'fused attention vs oracle parts={parts} pos={pos}')
    qkv = torch.randn(3 * H * D, generator=g).half()
    inv = (1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))).half()
    inv_freq = torch.cat([inv, inv])
    kc = (torch.randn(S, H * D, generator=g) * 0.5).half()
    vc = torch.randn(S, H * D, generator=g).half()
    att_f = 1 / math.sqrt(D)
    # oracle: rotate q and k, put k and v into row `pos`, attend over rows 0..pos
    q, k, v = qkv[:H * D].numpy(), qkv[H * D:2 * H * D].numpy(), qkv[2 * H * D:].numpy()
    q_rot = hot_ops.rotary(q.reshape(H, 2, D // 2), inv_freq.numpy(), pos)
    k_rot = hot_ops.rotary(k.reshape(H, 2, D // 2), inv_freq.numpy(), pos)
    kc_want, vc_want = kc.numpy().copy(), vc.numpy().copy()
    kc_want[pos], vc_want[pos] = k_rot.reshape(-1), v
    att_want = hot_ops.attention(q_rot, kc_want[:pos + 1].reshape(pos + 1, H, D), vc_want[:pos + 1].reshape(pos + 1, H, D), att_f)

    kd, vd = kc.to(dev), vc.to(dev)
    att_f_t = torch.tensor([att_f], dtype=torch.float32, device=dev)
    pos_t = torch.tensor([pos], dtype=torch.int32, device=dev)
    if parts == 1:
        att = torch.empty(H, D, dtype=torch.float16, device=dev)
        autort.ops.attention_rope_f16(qkv.to(dev), inv_freq.to(dev), kd, vd, att_f_t, att, extra=[pos_t])
        assert np.allclose(att.float().cpu().numpy(), att_want.astype(np.float32), **FP16_TOL)
    else:
        p = workloads.w4_problem(11, 1, H * D, 4096)
        res = torch.randn(4096, generator=g).half()
        partial = torch.full((H, parts, 132), float('nan'), dtype=torch.float32, device=dev)
        autort.ops.attention_rope_split_f16(qkv.to(dev), inv_freq.to(dev), kd, vd, att_f_t, partial, extra=[pos_t])
        y = torch.empty(4096, dtype=torch.float16, device=dev)
        autort.ops.gemv_w4a16_attn(partial, p['qweight'].to(dev), p['scales'].to(dev), p['qzeros'].to(dev), y, residual=res.to(dev))
        proj = hot_ops.gemm_w4a16(att_want.reshape(1, -1), p['qweight'].numpy(), p['scales'].numpy(), p['qzeros'].numpy()).reshape(-1)
        y_want = (proj.astype(np.float32) + res.numpy().astype(np.float32)).astype(np.float16)
        assert np.allclose(y.float().cpu().numpy(), y_want.astype(np.float32), **FP16_TOL)
    # cache: row `pos` rewritten, every other row untouched (bit for bit)
    kg, vg = kd.cpu().numpy(), vd.cpu().numpy()
    assert np.allclose(kg[pos].astype(np.float32), kc_want[pos].astype(np.float32), **FP16_TOL)
    assert np.array_equal(vg[pos], vc_want[pos])
    keep = np.arange(S) != pos
    assert np.array_equal(kg[keep], kc.numpy()[keep]) and np.array_equal(vg[keep], vc.numpy()[keep])


@pytest.mark.usefixtures('oracle_built')
@pytest.mark.parametrize('T,H', [(1, 4), (5, 4), (31, 4), (32, 32), (33, 4), (100, 32), (128, 32), (200, 4), (384, 32)])
def test_causal_attention_over_a_prompt_against_the_oracle(T, H):
    """attention_causal_f16 (matrix cores, one wavefront per 32 queries) against the oracle's attention applied position by
    position: query t sees rows 0..t of cache views that have more rows than the prompt."""
    import autort
    from oracle import hot_ops
    dev = autort.device()
    D, S = 128, T + 7
    g = torch.Generator().manual_seed(31 * T + H)
    note(f'causal attention T={T} H={H}')
    q = torch.randn(T, H, D, generator=g).half()
    kc = (torch.randn(S, H * D, generator=g) * 0.7).half()
    vc = torch.randn(S, H * D, generator=g).half()
    att_f = 1 / math.sqrt(D)
    out = autort.ops.attention_causal_f16(q.to(dev), kc.to(dev).view(S, H, D), vc.to(dev).view(S, H, D),
                                          torch.tensor([att_f], dtype=torch.float32, device=dev)).cpu().numpy()
    assert out.shape == (T, H, D)
    ks, vs = kc.numpy().reshape(S, H, D), vc.numpy().reshape(S, H, D)
    for t in sorted({0, 1, T // 3, T // 2, T - 2, T - 1} & set(range(T))) if T > 40 else range(T):
        want = hot_ops.attention(q[t].numpy(), ks[:t + 1], vs[:t + 1], att_f)
        assert np.allclose(out[t].astype(np.float32), want.astype(np.float32), **FP16_TOL), (t, np.abs(out[t].astype(np.float32) - want.astype(np.float32)).max())
    # the probabilities are rounded to fp16 before they meet V: compare every position with float64 as well
    qd, kd, vd = q.double(), kc.double().view(S, H, D), vc.double().view(S, H, D)
    sc = torch.einsum('thd,shd->hts', qd, kd[:T]) * att_f
    sc = sc.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float('-inf'))
    exact = torch.einsum('hts,shd->thd', torch.softmax(sc, -1), vd[:T]).numpy()
    assert np.allclose(out.astype(np.float64), exact, rtol=1e-2, atol=1e-2)


@pytest.mark.usefixtures('oracle_built')
def test_rope_qkv_store_rows_against_the_oracle():
    """The prompt form of rope_qkv_store: row t rotated at position first_pos + t, k and v into those cache rows."""
    import autort
    from oracle import hot_ops
    dev = autort.device()
    T, H, D, S, first = 9, 4, 128, 20, 3
    g = torch.Generator().manual_seed(77)
    note('rope_qkv_store_rows')
    qkv = torch.randn(T, 3 * H * D, generator=g).half()
    inv = (1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))).half()
    inv_freq = torch.cat([inv, inv])
    kc = torch.randn(S, H * D, generator=g).half()
    vc = torch.randn(S, H * D, generator=g).half()
    kd, vd = kc.to(dev), vc.to(dev)
    q_out = torch.zeros(T, H, D, dtype=torch.float16, device=dev)
    autort.ops.rope_qkv_store_rows_f16(qkv.to(dev), inv_freq.to(dev), q_out, kd, vd, extra=[first])
    for t in range(T):
        q, k, v = qkv[t, :H * D].numpy(), qkv[t, H * D:2 * H * D].numpy(), qkv[t, 2 * H * D:].numpy()
        want_q = hot_ops.rotary(q.reshape(H, 2, D // 2), inv_freq.numpy(), first + t)
        want_k = hot_ops.rotary(k.reshape(H, 2, D // 2), inv_freq.numpy(), first + t)
        assert np.allclose(q_out[t].float().cpu().numpy(), want_q.astype(np.float32), **FP16_TOL)
        assert np.allclose(kd[first + t].float().cpu().numpy(), want_k.reshape(-1).astype(np.float32), **FP16_TOL)
        assert np.array_equal(vd[first + t].cpu().numpy(), v)
    keep = [s for s in range(S) if not first <= s < first + T]
    assert torch.equal(kd.cpu()[keep], kc[keep]) and torch.equal(vd.cpu()[keep], vc[keep])
    # positions that do not fit the caches are refused on the host
    with pytest.raises(Exception, match='do not fit'):
        autort.ops.rope_qkv_store_rows_f16(qkv.to(dev), inv_freq.to(dev), q_out, kd, vd, extra=[S - T + 1])


def _tile_sums_of_squares(y: torch.Tensor) -> np.ndarray:
    """What a projection leaves in its sum-of-squares buffer for the fp16 outputs y: per tile of 128 columns the sum of
    floor(y^2 * 2^30), each square capped at 2^25 (integer arithmetic)."""
    sq = y.double().cpu().numpy() ** 2
    fixed = np.where(sq < 2.0 ** 25, np.floor(sq * 2.0 ** 30), 2.0 ** 55).astype(np.uint64)
    pad = (-fixed.size) % 128
    return np.concatenate([fixed, np.zeros(pad, dtype=np.uint64)]).reshape(-1, 128).sum(axis=1)


@pytest.mark.parametrize('K,N,scale', [(1024, 512, 1.0), (4096, 4096, 1.0), (11008, 4096, 0.02), (512, 272, 300.0)])
def test_sum_of_squares_handed_from_one_projection_to_the_next(autort, K, N, scale):
    """The projection that writes a residual stream (with residual add, plain or SwiGLU input) leaves sum(y^2) per
    column tile as exact integers and zeroes the other buffer; the projection that normalises the stream and takes the
    sum from the buffer agrees with the one that computes it from x, and with the oracle."""
    from oracle import hot_ops
    from antares_amd import workloads
    dev = autort.device()
    note(f'sum of squares K={K} N={N} scale={scale}')
    g = gen(K + N)
    p = workloads.w4_problem(K + 3 * N, 1, K, N)
    qw, sc, qz = (p[k].to(dev) for k in ('qweight', 'scales', 'qzeros'))
    x = (torch.randn(K, generator=g) * scale).half().to(dev)
    res = (torch.randn(N, generator=g) * scale).half().to(dev)
    a = torch.zeros(256, dtype=torch.int64, device=dev)
    b = torch.full((256,), 12345, dtype=torch.int64, device=dev)
    y = autort.ops.gemv_w4a16_fused(x, qw, sc, qz, residual=res, sumsq_out=a, sumsq_clear=b)
    y_plain = autort.ops.gemv_w4a16_fused(x, qw, sc, qz, residual=res)
    torch.cuda.synchronize()
    assert torch.equal(y, y_plain)
    assert int(b.abs().max()) == 0
    want = _tile_sums_of_squares(y)
    got = a.cpu().numpy().astype(np.uint64)
    assert np.array_equal(got[:want.size], want) and not got[want.size:].any()
    # a second writer adds on top (the decoder clears in between)
    autort.ops.gemv_w4a16_fused(x, qw, sc, qz, residual=res, sumsq_out=a)
    torch.cuda.synchronize()
    assert np.array_equal(a.cpu().numpy().astype(np.uint64)[:want.size], 2 * want)
    a.zero_()
    a[:want.size] = torch.from_numpy(want.astype(np.int64)).to(dev)
    # the consumer: y is the stream (N must be a K of its own: a multiple of 128 here except in the ragged case)
    if N % 128:
        return
    p2 = workloads.w4_problem(N + 5, 1, N, 528)
    qw2, sc2, qz2 = (p2[k].to(dev) for k in ('qweight', 'scales', 'qzeros'))
    nw = (torch.rand(N, generator=g) + 0.5).half().to(dev)
    handed = autort.ops.gemv_w4a16_fused(y, qw2, sc2, qz2, norm_weight=nw, eps=1e-5, sumsq_in=a)
    own = autort.ops.gemv_w4a16_fused(y, qw2, sc2, qz2, norm_weight=nw, eps=1e-5)
    torch.cuda.synchronize()
    assert torch.allclose(handed.float(), own.float(), rtol=2e-3, atol=2e-3)
    xn = hot_ops.rmsnorm(y.cpu().numpy(), None, nw.cpu().numpy(), 1.0 / N, 1e-5, np.float16)
    ref = hot_ops.gemm_w4a16(xn.reshape(1, -1), p2['qweight'].numpy(), p2['scales'].numpy(), p2['qzeros'].numpy())
    assert np.allclose(handed.cpu().numpy().astype(np.float32).reshape(1, -1), ref.astype(np.float32), **FP16_TOL)


def test_sum_of_squares_through_the_attention_merge(autort):
    """gemv_w4a16_attn leaves the same sums as the fused projection on the merged attention output."""
    from antares_amd import workloads
    dev = autort.device()
    H, D, S, parts, pos = 32, 128, 384, 8, 200
    g = gen(77)
    qkv = torch.randn(3 * H * D, generator=g).half().to(dev)
    inv = (1.0 / (10000 ** (torch.arange(0, D, 2).float() / D))).half()
    inv_freq = torch.cat([inv, inv]).to(dev)
    kc = (torch.randn(S, H * D, generator=g) * 0.5).half().to(dev)
    vc = torch.randn(S, H * D, generator=g).half().to(dev)
    att_f = torch.tensor([1 / math.sqrt(D)], dtype=torch.float32, device=dev)
    pos_t = torch.tensor([pos], dtype=torch.int32, device=dev)
    p = workloads.w4_problem(9, 1, H * D, 4096)
    qw, sc, qz = (p[k].to(dev) for k in ('qweight', 'scales', 'qzeros'))
    res = torch.randn(4096, generator=g).half().to(dev)
    partial = torch.full((H, parts, 132), float('nan'), dtype=torch.float32, device=dev)
    autort.ops.attention_rope_split_f16(qkv, inv_freq, kc, vc, att_f, partial, extra=[pos_t])
    a = torch.zeros(256, dtype=torch.int64, device=dev)
    b = torch.ones(256, dtype=torch.int64, device=dev)
    y = torch.empty(4096, dtype=torch.float16, device=dev)
    autort.ops.gemv_w4a16_attn(partial, qw, sc, qz, y, residual=res, sumsq_out=a, sumsq_clear=b)
    torch.cuda.synchronize()
    want = _tile_sums_of_squares(y)
    assert np.array_equal(a.cpu().numpy().astype(np.uint64)[:32], want) and int(b.abs().max()) == 0


def test_sum_of_squares_buffers_are_checked(autort):
    from antares_amd.runtime import capi
    from antares_amd import workloads
    dev = autort.device()
    p = workloads.w4_problem(3, 1, 256, 256)
    qw, sc, qz = (p[k].to(dev) for k in ('qweight', 'scales', 'qzeros'))
    x = torch.randn(256).half().to(dev)
    a = torch.zeros(256, dtype=torch.int64, device=dev)
    with pytest.raises(capi.ArtError, match='norm weight'):
        autort.ops.gemv_w4a16_fused(x, qw, sc, qz, sumsq_in=a)
    with pytest.raises(capi.ArtError, match='cannot be the one'):
        autort.ops.gemv_w4a16_fused(x, qw, sc, qz, sumsq_out=a, sumsq_clear=a)
    with pytest.raises(TypeError, match='sum-of-squares buffer'):
        autort.ops.gemv_w4a16_fused(x, qw, sc, qz, sumsq_out=torch.zeros(8, dtype=torch.int64, device=dev))
