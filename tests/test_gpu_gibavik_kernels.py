"""The kernels that came with Gibavik, each against a plain PyTorch float32 form of the same operation: the three
attention kernels with capped scores and a distance term a head (single tokens through chunks of keys, portions in
query tiles whole and cut by keys, the float kernel), the scan of a memory that fades by a constant a head at key
sizes on either side of the scan's switches, the sum of scaled terms behind a norm into the stream with its copy,
the norm over runs of columns with rows of zeros between the values, the turn of heads by position with and without
a gate, the stream as an operand, the experts' table, the bounded gate activation. Several requests of unequal length
in one call, calls that go on from the state the calls before left, a request that starts afresh in a slot that was
used, and padding rows (state slot -1) that must leave every state alone."""
import math

import pytest
import torch

from kernel_double import KernelDouble
from reinfer_amd import kernels
from test_gpu_detatar_kernels import CALLS, close, make_batch
from test_gpu_kernels import DEC_BATCHES, DT, PRE_BATCHES, FakeBatch, kt, make_paged_case, vt

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ------------------------------------------------------------------ attention with changed scores
def changed_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window, cap, r1, r2):
    """Every query against its request's keys, gathered through the block table, in double precision."""
    bs = kc.shape[2]
    out, t0 = [], 0
    for i, (ql, st) in enumerate(zip(q_lens, starts)):
        n = st + ql
        keys = torch.arange(n)
        blk = tables[i, keys // bs].long().cpu()
        K = torch.nan_to_num(kc.double().cpu()[blk, :, keys % bs, :])       # [n, Hkv, d]
        V = torch.nan_to_num(vc.double().cpu()[blk, :, keys % bs, :])
        for j in range(ql):
            p = st + j
            lo = max(0, p - window + 1) if window else 0
            row = []
            for a in range(Hq):
                g = a // (Hq // Hkv)
                s = (K[lo:p + 1, g] @ q[t0 + j, a].double().cpu()) * scale
                if cap:
                    s = cap * torch.tanh(s / cap)
                if r1 is not None:
                    s = s - float(r1[a]) * torch.log(1.0 + float(r2[a]) * (p - torch.arange(lo, p + 1)).double())
                row.append(torch.softmax(s, 0) @ V[lo:p + 1, g])
            out.append(torch.cat(row))
        t0 += ql
    return torch.stack(out)


def score_changes(Hq, seed):
    g = torch.Generator().manual_seed(seed)
    r1 = (0.3 + 1.5 * torch.rand(Hq, generator=g)).to(DEV)
    r2 = (0.05 + 0.5 * torch.rand(Hq, generator=g)).to(DEV)
    return [(2.5, None), (0.0, (r1, r2)), (4.0, (r1, r2))]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,Hkv,d", [(4, 2, 16), (6, 3, 96), (5, 5, 32), (8, 1, 128), (3, 1, 48)])
def test_attention_plain_with_changed_scores(dtype, Hq, Hkv, d):
    ops = kernels.current()
    for bi, (q_lens, starts) in enumerate([([1, 1, 1], [31, 32, 300]), ([2, 17, 1, 40], [0, 30, 99, 1])]):
        for window in (0, 19):
            for cap, dist in score_changes(Hq, bi):
                q, kc, vc, tables = make_paged_case(dtype, Hq, Hkv, d, q_lens, starts, seed=bi)
                batch = FakeBatch(q_lens, starts, tables)
                T = sum(q_lens)
                out = torch.empty(T, Hq * d, device=DEV, dtype=DT[dtype])
                scale = 2.0 / math.sqrt(d)
                ops.attention_plain(q.view(T, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window, 0,
                                    mod=ops._score_mod(cap, dist, Hq, q.device))
                ref = changed_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window, cap,
                                        dist[0] if dist else None, dist[1] if dist else None)
                close(out, ref, 2e-5 if dtype == "float32" else 2 ** -7, (bi, window, cap))


@pytest.mark.parametrize("Hq,Hkv,d", [(4, 2, 16), (6, 3, 96), (6, 2, 64), (8, 1, 128), (16, 1, 32), (3, 3, 48), (2, 1, 256)])
def test_attention_decode_with_changed_scores(Hq, Hkv, d):
    ops = kernels.current()
    for bi, (q_lens, starts) in enumerate(DEC_BATCHES[:5]):
        for window in (0, 19, 150):
            for cap, dist in score_changes(Hq, 10 + bi):
                for chunk, waves in ((None, None), (128, 4), (256, 12)):
                    q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=10 + bi)
                    batch = FakeBatch(q_lens, starts, tables)
                    T = sum(q_lens)
                    out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
                    scale = 2.0 / math.sqrt(d)
                    ops.attention_decode(q.view(T, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window,
                                         0, chunk=chunk, waves=waves, mod=ops._score_mod(cap, dist, Hq, q.device))
                    ref = changed_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window, cap,
                                            dist[0] if dist else None, dist[1] if dist else None)
                    close(out, ref, 2 ** -7, (bi, window, cap, chunk))


@pytest.mark.parametrize("Hq,Hkv,d", [(4, 2, 16), (6, 3, 96), (6, 2, 64), (8, 1, 128), (3, 3, 48), (2, 1, 256)])
def test_attention_prefill_with_changed_scores(Hq, Hkv, d):
    ops = kernels.current()
    tile = kernels.library.load().ra_attention_prefill_tile(Hq, Hkv, d)
    for bi, (q_lens, starts) in enumerate(PRE_BATCHES[:5]):
        for window in (0, 19, 150):
            for cap, dist in score_changes(Hq, 20 + bi):
                q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=20 + bi)
                batch = FakeBatch(q_lens, starts, tables)
                T = sum(q_lens)
                info, t = [], 0
                for i, (ql, st) in enumerate(zip(q_lens, starts)):
                    for q0 in range(0, ql, tile):
                        info += [i, t + q0, min(tile, ql - q0), st + q0]
                    t += ql
                tiles = torch.tensor(info, dtype=torch.int32, device=DEV)
                scale = 2.0 / math.sqrt(d)
                mod = ops._score_mod(cap, dist, Hq, q.device)
                out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
                ops.attention_prefill(q.view(T, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window, 0,
                                      tiles, len(info) // 4, mod=mod)
                ref = changed_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window, cap,
                                        dist[0] if dist else None, dist[1] if dist else None)
                close(out, ref, 2 ** -7, (bi, window, cap))
                # every other tile cut by keys into parts of two rounds of 64, added by the second kernel
                items, merge, n_slots = [], [], 0
                for k in range(len(info) // 4):
                    i, row, n, pos = info[4 * k:4 * k + 4]
                    parts = -(-(-(-(pos + n) // 64)) // 2)
                    if k % 2 == 1 or parts < 2:
                        items.append(((i, row, n, pos), (0, 1 << 30, -1)))
                        continue
                    merge += [row, n, n_slots, parts]
                    for c in range(parts):
                        items.append(((i, row, n, pos), (c * 128, (c + 1) * 128 if c + 1 < parts else 1 << 30, n_slots + c)))
                    n_slots += parts
                if merge:
                    out2 = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
                    ops.attention_prefill(q.view(T, Hq * d), Hq * d, out2, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window, 0,
                                          torch.tensor([v for it in items for v in it[0]], dtype=torch.int32, device=DEV),
                                          len(items),
                                          torch.tensor([v for it in items for v in it[1]], dtype=torch.int32, device=DEV),
                                          torch.tensor(merge, dtype=torch.int32, device=DEV), len(merge) // 4, n_slots, mod=mod)
                    close(out2, ref, 2 ** -7, (bi, window, cap, "cut"))


def test_attention_dispatch_passes_the_changes_on():
    """A mixed step (single tokens beside portions) through ``attention``: whatever kernels it picks, the cap and
    the distance term are in the result."""
    ops = kernels.current()
    Hq, Hkv, d = 6, 3, 96
    q_lens, starts = [1, 70, 1, 3, 200], [260, 0, 17, 40, 100]
    cap, dist = score_changes(Hq, 3)[2]
    for dtype in ("bfloat16", "float32"):
        q, kc, vc, tables = make_paged_case(dtype, Hq, Hkv, d, q_lens, starts, seed=5)
        batch = FakeBatch(q_lens, starts, tables)
        T = sum(q_lens)
        out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=DT[dtype])
        ops.attention(q.view(T, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, 0.2, 50, 0, softcap=cap,
                      distance=dist)
        ref = changed_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, 0.2, 50, cap, dist[0], dist[1])
        close(out, ref, 2 ** -7 if dtype == "bfloat16" else 2e-5, dtype)
        plain_out = torch.empty_like(out)
        ops.attention(q.view(T, Hq * d), Hq * d, plain_out, kt(kc), vt(vc), batch, Hq, Hkv, d, 0.2, 50, 0)
        assert float((plain_out.float() - out.float()).abs().max()) > 0.05       # the changes are not small here


# ------------------------------------------------------------------ the fading memory
@pytest.mark.parametrize("H,dk,dv", [(2, 32, 32), (3, 20, 12), (1, 136, 8), (4, 64, 32), (1, 8, 40), (5, 12, 12),
                                     (2, 4, 6), (1, 40, 8), (2, 128, 64), (1, 300, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decay_scan(H, dk, dv, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(H * 1000 + dk)
    nk, nv = H * dk, H * dv
    width = 2 * nk + nv + 9
    q_off, k_off, v_off = 2, 2 + nk, 5 + 2 * nk
    decays = torch.rand(H, generator=g) * 0.6 + 0.399
    st_gpu = torch.full((4, ops.scan_state_floats("decay_memory", H, dk, dv) + 3), float("nan"), device=DEV)
    st_ref = torch.full((4, ref.scan_state_floats("decay_memory", H, dk, dv) + 3), float("nan"))
    for i, (q_lens, slots, fresh) in enumerate(CALLS):
        T = sum(q_lens)
        proj = (torch.randn(T, width, generator=g) * 0.9).to(dtype)
        out_ref = torch.empty(T, nv)
        ref.decay_scan(proj, q_off, k_off, v_off, decays, st_ref, make_batch(q_lens, slots, fresh, "cpu"), H, dk, dv, out_ref)
        out = torch.empty(T, nv, device=DEV)
        before = st_gpu.clone()
        ops.decay_scan(proj.to(DEV), q_off, k_off, v_off, decays.to(DEV), st_gpu, make_batch(q_lens, slots, fresh, DEV),
                       H, dk, dv, out)
        close(out, out_ref, 2e-5, f"call {i}")
        untouched = [s for s in range(4) if s not in slots]
        assert torch.equal(torch.nan_to_num(st_gpu[untouched], nan=7.0), torch.nan_to_num(before[untouched], nan=7.0))
        assert torch.isnan(st_gpu[:, -3:]).all()


def test_decay_scan_by_hand():
    """One head, keys of two, three tokens, no silu to speak of (large inputs pass it nearly unchanged): the
    read-out sees the token's own write, the factor fades what came before."""
    ops = kernels.current()
    big = 40.0                                            # silu(40 x) = 40 x for x > 0 to float precision
    q = torch.tensor([[1.0, 1.0], [1.0, 0.5], [0.5, 1.0]]) * big
    k = torch.tensor([[1.0, 2.0], [1.0, 1.0], [3.0, 1.0]]) * big
    v = torch.tensor([[1.0], [2.0], [0.5]]) * big
    proj = torch.cat([q, k, v], dim=1).to(DEV)
    state = torch.zeros(1, ops.scan_state_floats("decay_memory", 1, 2, 1), device=DEV)
    out = torch.empty(3, 1, device=DEV)
    dec = 0.5
    ops.decay_scan(proj, 0, 2, 4, torch.tensor([dec], device=DEV), state, make_batch([3], [0], [1], DEV), 1, 2, 1, out)
    S = torch.zeros(2)
    want = []
    for t in range(3):
        S = dec * S + k[t] * v[t, 0]
        want.append(float(S @ q[t]))
    close(out.view(-1), torch.tensor(want), 1e-6, "by hand")


# ------------------------------------------------------------------ rows
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("h", [36, 64, 256, 4096, 9000])
def test_sum_norm_add_and_stream_cast(dtype, h):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(h)
    T = 7
    for n, in_dtype in ((1, torch.float32), (2, torch.float32), (1, dtype), (3, dtype)):
        xs = [(torch.randn(T, h, generator=g) * (i + 1)).to(in_dtype) for i in range(n)]
        scales = [0.7, 1.1, -1.5][:n]
        for weight in (torch.tensor([1.7]), torch.rand(h, generator=g) + 0.5, None):
            for with_resid, with_copy in ((True, True), (True, False), (False, True)):
                resid = torch.randn(T, h, generator=g)
                r_ref, r_gpu = resid.clone(), resid.to(DEV)
                c_ref = torch.empty(T, h, dtype=dtype) if with_copy else None
                c_gpu = torch.empty(T, h, dtype=dtype, device=DEV) if with_copy else None
                ref.sum_norm_add(xs, scales, weight, 1e-5, resid=r_ref if with_resid else None, copy=c_ref)
                ops.sum_norm_add([x.to(DEV) for x in xs], scales, weight.to(DEV) if weight is not None else None, 1e-5,
                                 resid=r_gpu if with_resid else None, copy=c_gpu)
                if with_resid:
                    close(r_gpu, r_ref, 2e-6, (n, "stream"))
                else:
                    assert torch.equal(r_gpu.cpu(), resid)
                if with_copy:
                    close(c_gpu, c_ref, 2e-6 if dtype == torch.float32 else 2 ** -8, (n, "copy"))
    x = torch.randn(T, h, generator=g)
    out = torch.empty(T, h, dtype=dtype, device=DEV)
    ops.stream_cast(x.to(DEV), out)
    assert torch.equal(out.cpu(), x.to(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_span_rmsnorm_counts_the_values_not_the_zeros_between_them(dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(3)
    T, H, G, D, dk = 9, 3, 2, 32, 24
    width = (H + 2 * G) * D
    x = torch.randn(T, width, generator=g)
    x.view(T, H + 2 * G, D)[:, :, dk:] = 0                  # rows of zeros behind each head's values
    x = x.to(dtype)
    wq, wk = torch.rand(H * D, generator=g) + 0.5, torch.rand(G * D, generator=g) + 0.5
    spans = [(0, H * D, wq, H * dk), (H * D, G * D, wk, G * dk)]
    want = x.clone()
    ref.span_rmsnorm(want, spans, 1e-5)
    got = x.to(DEV)
    ops.span_rmsnorm(got, [(c, w, wt.to(DEV), n) for c, w, wt, n in spans], 1e-5)
    close(got, want, 2e-6 if dtype == torch.float32 else 2 ** -8, "two runs")
    assert torch.equal(got[:, (H + G) * D:].cpu(), x[:, (H + G) * D:])          # the values' columns are left alone
    # by hand: the mean is over the 72 values, not the 96 columns
    v = x[0, :H * D].double()
    assert torch.allclose(want[0, :H * D].double(), (v / torch.sqrt((v * v).sum() / (H * dk) + 1e-5) * wq.double()).to(dtype).double())
    one = x.to(DEV)
    ops.span_rmsnorm(one, [(0, H * D, wq.to(DEV), H * dk)], 1e-5)
    assert torch.equal(one[:, H * D:].cpu(), x[:, H * D:])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("style", [0, 1])
def test_turn_heads(dtype, style):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(4 + style)
    T = 11
    pos = torch.randint(0, 3000, (T,), generator=g).to(torch.int32)
    for heads, stride, width in ((3, 32, 24), (2, 16, 16), (5, 48, 2), (1, 64, 0)):
        inv = (10000.0 ** (-2.0 * torch.arange(max(width // 2, 1)).double() / max(width, 1))).float()
        lead, tail = 5, 7
        buf = torch.randn(T, lead + heads * stride + tail, generator=g).to(dtype)
        gate = torch.randn(T, heads * stride + 3, generator=g).to(dtype)
        for sign, with_gate in ((1.0, False), (-1.0, True), (-1.0, False)):
            if width == 0 and not with_gate:
                continue
            want, got = buf.clone(), buf.to(DEV)
            ref.turn_heads(want[:, lead:lead + heads * stride], heads, stride, width, style, pos, inv, sign,
                           gate=gate if with_gate else None, gate_stride=stride)
            ops.turn_heads(got[:, lead:lead + heads * stride], heads, stride, width, style, pos.to(DEV), inv.to(DEV), sign,
                           gate=gate.to(DEV) if with_gate else None, gate_stride=stride)
            close(got, want, 1e-5 if dtype == torch.float32 else 2 ** -7, (heads, stride, width, sign, with_gate))
            assert torch.equal(got[:, :lead].cpu(), buf[:, :lead]) and torch.equal(got[:, -tail:].cpu(), buf[:, -tail:])
    # there and back is the identity, and a turn by position p then by q is one by p + q in effect: by hand for a pair
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV)
    ops.turn_heads(x, 1, 4, 4, style, torch.tensor([2], dtype=torch.int32, device=DEV), torch.tensor([0.5, 0.25], device=DEV), 1.0)
    pairs = ((0, 2), (1, 3)) if style == 0 else ((0, 1), (2, 3))
    src = [1.0, 2.0, 3.0, 4.0]
    for m, (a, b) in enumerate(pairs):
        ang = 2 * (0.5, 0.25)[m]
        assert abs(float(x[0, a]) - (src[a] * math.cos(ang) - src[b] * math.sin(ang))) < 1e-6
        assert abs(float(x[0, b]) - (src[b] * math.cos(ang) + src[a] * math.sin(ang))) < 1e-6


def test_experts_from_the_table_and_the_bounded_activation():
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(6)
    V, top, T = 50, 3, 13
    table = torch.stack([torch.randperm(7, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    toks = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    ids, wts = torch.empty(T, top, dtype=torch.int32, device=DEV), torch.empty(T, top, device=DEV)
    ops.moe_table_route(toks.to(DEV), table.to(DEV), ids, wts)
    assert torch.equal(ids.cpu(), table[toks.long()]) and torch.allclose(wts.cpu(), torch.full((T, top), 1.0 / 3.0))
    for dtype in (torch.float32, torch.bfloat16):
        for I, group in ((40, 8), (24, 0), (21, 0)):
            gu = (torch.randn(T, 2 * I, generator=g) * 2).to(dtype)
            want, got = torch.empty(T, I, dtype=dtype), torch.empty(T, I, dtype=dtype, device=DEV)
            ref.silu_mul(gu, want, group, act="swish_bounded", limit=1.25)
            ops.silu_mul(gu.to(DEV), got, group, act="swish_bounded", limit=1.25)
            close(got, want, 2e-6 if dtype == torch.float32 else 2 ** -8, (I, group))
    with pytest.raises(ValueError):
        ops.silu_mul(gu.to(DEV), got, 0, act="swish_bounded")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,dv", [(1, 4096), (1, 520), (3, 512), (1, 96), (2, 9000)])
def test_head_norm_gate_over_wide_heads(dtype, H, dv):
    """One norm over all read-outs of a row (a single head as wide as all of them), and heads wide enough for the
    form that gives a workgroup to each."""
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(dv)
    T, n = 5, H * dv
    read = torch.randn(T, n, generator=g) * 3
    weight = torch.rand(n, generator=g) + 0.5
    gate = torch.randn(T, n + 16, generator=g).to(dtype)
    for kind in ("sigmoid", "silu"):
        want = torch.empty(T, n, dtype=dtype)
        ref.head_norm_gate(read, weight, True, gate, kind, 1e-5, H, dv, want)
        got = torch.empty(T, n, dtype=dtype, device=DEV)
        ops.head_norm_gate(read.to(DEV), weight.to(DEV), True, gate.to(DEV), kind, 1e-5, H, dv, got)
        close(got, want, 2e-6 if dtype == torch.float32 else 2 ** -8, (H, dv, kind))
