"""The kernels that came with Detatar, each against a plain PyTorch float32 form of the same operation (the CPU
stand-in's, which has the same signature and shares no code with the product): the wkv scan at head sizes on either
side of the scan's switches (8, 16 or more lanes a column), the mix with the row before in one and in five mixes,
the gated add into the stream, the norm in groups, the tanh form of the gated activation, the softmax router with
its correction, groups and identity experts, the head products with one gate a head. Several requests of unequal
length in one call, calls that go on from the state the calls before left, a request that starts afresh in a slot
that was used, steps of single tokens, and padding rows (state slot -1) that must leave every state alone."""
from types import SimpleNamespace

import pytest
import torch

from kernel_double import KernelDouble
from reinfer_amd import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_batch(q_lens, slots, fresh, device):
    cu = [0]
    for q in q_lens:
        cu.append(cu[-1] + q)
    seq_of = [i for i, q in enumerate(q_lens) for _ in range(q)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return SimpleNamespace(num_seqs=len(q_lens), num_tokens=cu[-1], cu_tokens=i32(cu), state_slots=i32(slots),
                           fresh=i32(fresh), seq_of_token=i32(seq_of), q_lens=list(q_lens), max_q_len=max(q_lens))


# slots 2 and 0 start; they go on beside a padding row, one token each; slot 2 starts afresh beside slot 0 going on;
# portions of several staged chunks, the last of them part full; single tokens again
CALLS = [([5, 3], [2, 0], [1, 1]), ([1, 1, 1], [2, -1, 0], [0, 0, 0]), ([7, 2], [2, 0], [1, 0]),
         ([53, 1, 40], [0, 3, 2], [0, 1, 0]), ([1, 1, 1], [3, 0, 2], [0, 0, 0])]


def close(got, ref, tol, what):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert torch.isfinite(got).all(), what
    err = float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-20))
    assert err < tol, (what, err)


@pytest.mark.parametrize("H,d", [(2, 32), (3, 20), (1, 136), (2, 64), (1, 8), (5, 12), (2, 4), (4, 9), (1, 40), (2, 128)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_wkv_scan(H, d, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(H * 1000 + d)
    n = H * d
    width = 3 * n + 9
    r_off, k_off, v_off = 2, 2 + n, 4 + 2 * n
    w0 = torch.rand(n, generator=g) * 3.0 - 2.5
    u = torch.randn(n, generator=g) * 0.5
    st_gpu = torch.full((4, ops.scan_state_floats("wkv", H, d, d) + 3), float("nan"), device=DEV)
    st_ref = torch.full((4, ref.scan_state_floats("wkv", H, d, d) + 3), float("nan"))
    for i, (q_lens, slots, fresh) in enumerate(CALLS):
        T = sum(q_lens)
        proj = (torch.randn(T, width, generator=g) * 0.7).to(dtype)
        z = torch.randn(T, n + 5, generator=g)                       # decays' pre-activations, rows wider than needed
        out_ref = torch.empty(T, n)
        ref.wkv_scan(proj, r_off, k_off, v_off, z.clone(), w0, u, st_ref, make_batch(q_lens, slots, fresh, "cpu"), H, d, out_ref)
        out = torch.empty(T, n, device=DEV)
        before = st_gpu.clone()
        ops.wkv_scan(proj.to(DEV), r_off, k_off, v_off, z.to(DEV), w0.to(DEV), u.to(DEV), st_gpu,
                     make_batch(q_lens, slots, fresh, DEV), H, d, out)
        close(out, out_ref, 2e-5, f"call {i}")
        untouched = [s for s in range(4) if s not in slots]
        assert torch.equal(torch.nan_to_num(st_gpu[untouched], nan=7.0), torch.nan_to_num(before[untouched], nan=7.0))
        # behind the scan's own floats the slot belongs to someone else
        assert torch.isnan(st_gpu[:, -3:]).all()


def test_wkv_bonus_decay_and_order_by_hand():
    """One head of two channels, three tokens: the bonus for the current token alone, the decay of a token applied
    after its own read-out and write."""
    ops = kernels.current()
    H, d = 1, 2
    r = torch.tensor([[1.0, 1.0], [1.0, 0.0], [0.0, 1.0]])
    k = torch.tensor([[1.0, 2.0], [1.0, 1.0], [3.0, 1.0]])
    v = torch.tensor([[1.0, -1.0], [2.0, 0.5], [0.0, 1.0]])
    proj = torch.cat([r, k, v], dim=1).to(DEV)
    w = torch.tensor([[0.5, 0.25], [0.1, 0.2], [0.9, 0.9]])
    z = torch.log(-torch.log(w)).to(DEV)                            # exp(-exp(z)) = w, with w0 = 0
    u = torch.tensor([2.0, 3.0], device=DEV)
    st = torch.full((1, ops.scan_state_floats("wkv", H, d, d)), float("nan"), device=DEV)
    out = torch.empty(3, 2, device=DEV)
    ops.wkv_scan(proj, 0, 2, 4, z, torch.zeros(2, device=DEV), u, st, make_batch([3], [0], [1], DEV), H, d, out)
    # t0: S = 0: o = v0 * (u . k0 * r0) = v0 * (2 * 1 + 3 * 2) = 8 v0
    # S0 = k0 v0^T (decay w0 acts on the empty state)
    # t1: o = S0^T r1 + v1 * (u k1 . r1) = v0 * (k0 . r1) + v1 * 2 = v0 + 2 v1;  S1 = diag(w1) S0 + k1 v1^T
    # t2: o = S1^T r2 + v2 * (u k2 . r2) = v0 * (0.2 * 2) + v1 * 1 + v2 * 3
    want = torch.stack([8 * v[0], v[0] + 2 * v[1], 0.4 * v[0] + v[1] + 3 * v[2]])
    close(out, want, 1e-6, "by hand")


@pytest.mark.parametrize("width,n_mix,tail", [(64, 1, 2), (36, 5, 2), (200, 5, 2), (1024, 1, 2), (8, 2, 2), (64, 2, 8), (200, 5, 0),
                                              (4096, 5, 4), (1032, 3, 0), (2048, 1, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_shift(width, n_mix, tail, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(width + n_mix)
    mu = torch.rand(n_mix, width, generator=g).to(dtype)
    keep_off = 24
    # a state row of a whole number of 16 bytes (tail a multiple of 4 here) is read 16 bytes a thread
    st_gpu = torch.full((4, keep_off + width + tail), float("nan"), device=DEV)
    st_ref = torch.full((4, keep_off + width + tail), float("nan"))
    for i, (q_lens, slots, fresh) in enumerate(CALLS):
        T = sum(q_lens)
        wide = torch.randn(T, width + 8, generator=g).to(dtype)
        out_ref = torch.empty(T, n_mix * width, dtype=dtype)
        ref.token_shift(wide[:, 8:], mu, st_ref, keep_off, make_batch(q_lens, slots, fresh, "cpu"), out_ref)
        out = torch.empty(T, n_mix * width, dtype=dtype, device=DEV)
        ops.token_shift(wide.to(DEV)[:, 8:], mu.to(DEV), st_gpu, keep_off, make_batch(q_lens, slots, fresh, DEV), out)
        close(out, out_ref, 1e-6 if dtype == torch.float32 else 1e-2, f"call {i}")
        live = [s for s in slots if s >= 0]
        assert torch.equal(st_gpu[live, keep_off:keep_off + width].cpu(), st_ref[live, keep_off:keep_off + width]), i
        assert torch.isnan(st_gpu[:, :keep_off]).all() and torch.isnan(st_gpu[:, keep_off + width:]).all()


@pytest.mark.parametrize("width", [36, 64, 1000, 4096, 520])
@pytest.mark.parametrize("both", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_stream_add(width, both, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(width)
    T = 19
    resid = torch.randn(T, width, generator=g)
    gates = (torch.randn(T, 2 * width if both else width, generator=g) * 2).to(dtype)
    a = torch.randn(T, width, generator=g).to(dtype)
    b = torch.randn(T, width, generator=g).to(dtype) if both else None
    want = resid.clone()
    ref.gated_stream_add(want, gates, a, b)
    got = resid.to(DEV)
    ops.gated_stream_add(got, gates.to(DEV), a.to(DEV), b.to(DEV) if both else None)
    close(got, want, 1e-6, "stream")


@pytest.mark.parametrize("width,groups", [(64, 4), (36, 3), (192, 1), (1000, 8), (40, 5), (4096, 4), (2048, 1), (1536, 3),
                                          (8192, 2), (16384, 2), (2560, 10), (1792, 7)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_in_groups(width, groups, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(width)
    T = 13
    resid = torch.randn(T, width, generator=g) * torch.logspace(-1, 1, width)       # parts of very unequal size
    delta = torch.randn(T, width, generator=g).to(dtype)
    weight = torch.rand(width, generator=g) + 0.5
    rows = torch.tensor([12, 0, 5], dtype=torch.int32)
    for r in (None, rows):
        a, b = resid.clone(), resid.clone().to(DEV)
        n = T if r is None else 3
        out_ref, out = torch.empty(n, width, dtype=dtype), torch.empty(n, width, dtype=dtype, device=DEV)
        ref.add_rmsnorm(a, delta, weight, 1e-5, out_ref, r, groups=groups)
        ops.add_rmsnorm(b, delta.to(DEV), weight.to(DEV), 1e-5, out, None if r is None else r.to(DEV), groups=groups)
        close(out, out_ref, 1e-5 if dtype == torch.float32 else 1e-2, "norm")
        close(b, a, 1e-6, "stream")
    # the same by hand: each part over its own root mean square
    x = resid[:1]
    parts = x.view(1, groups, width // groups)
    want = (parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + 1e-5)).reshape(1, width) * weight
    out = torch.empty(1, width, device=DEV)
    ops.add_rmsnorm(x.clone().to(DEV), None, weight.to(DEV), 1e-5, out, groups=groups)
    close(out, want, 1e-5, "by hand")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rows_norm_tanh_and_gelu(dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(8)
    T = 21
    for width in (24, 80, 1536, 2048, 2056):
        wide = (torch.randn(T, width + 16, generator=g) * 3).to(dtype)
        weight = (torch.rand(width, generator=g) + 0.5).to(dtype)
        out_ref, out = torch.empty(T, width, dtype=dtype), torch.empty(T, width, dtype=dtype, device=DEV)
        ref.rows_rmsnorm(wide[:, 8:8 + width], weight, 1e-5, out_ref)
        ops.rows_rmsnorm(wide.to(DEV)[:, 8:8 + width], weight.to(DEV), 1e-5, out)
        close(out, out_ref, 1e-5 if dtype == torch.float32 else 1e-2, "rows_rmsnorm")
    x = (torch.randn(T, 37, generator=g) * 2).to(dtype)
    want, got = x.clone(), x.clone().to(DEV)
    ref.tanh_rows(want)
    ops.tanh_rows(got)
    close(got, want, 1e-6 if dtype == torch.float32 else 1e-2, "tanh")
    gu = (torch.randn(T, 2 * 88, generator=g) * 2).to(dtype)
    z, up = gu[:, :88].float(), gu[:, 88:].float()
    want = 0.5 * z * (1 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3))) * up
    out = torch.empty(T, 88, dtype=dtype, device=DEV)
    ops.silu_mul(gu.to(DEV), out, act="gelu_tanh")
    close(out, want, 1e-6 if dtype == torch.float32 else 1e-2, "gelu_tanh")


@pytest.mark.parametrize("E,top,groups,kept", [(8, 2, 4, 2), (10, 3, 2, 1), (6, 6, 1, 1), (64, 8, 8, 4), (9, 2, 9, 3), (130, 5, 2, 1),
                                               (3, 1, 1, 1), (1, 1, 1, 1)])
def test_moe_route_softmax(E, top, groups, kept):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(E)
    T, width = 37, 24
    x, router = torch.randn(T, width, generator=g), torch.randn(E + 1, width, generator=g) * 0.4
    corr = torch.randn(E, generator=g) * 0.1
    for c in (corr, None):
        ids_ref, w_ref = torch.empty(T, top, dtype=torch.int32), torch.empty(T, top)
        lg_ref = ref.moe_route(x, router, top, ids_ref, w_ref, scoring="softmax", groups=groups, groups_kept=kept,
                               correction=c, norm_eps=1e-20, outputs=E)
        ids, w = torch.empty(T, top, dtype=torch.int32, device=DEV), torch.empty(T, top, device=DEV)
        lg = ops.moe_route(x.to(DEV), router.to(DEV), top, ids, w, scoring="softmax", groups=groups, groups_kept=kept,
                           correction=None if c is None else c.to(DEV), norm_eps=1e-20, outputs=E)
        assert torch.equal(ids.cpu(), ids_ref)
        close(w, w_ref, 1e-5, "weights")
        close(lg, lg_ref, 1e-5, "logits")                        # the row behind the routed ones is the caller's


def test_moe_route_softmax_by_hand():
    """Scores made by hand. The correction decides the choice and stays out of the weights; a group is scored by
    its largest choice score; experts outside the kept groups cannot be chosen even where every choice score is
    negative; the weights are the chosen softmax scores over their sum."""
    ops = kernels.current()

    def route(z, corr, top, groups, kept):
        E = len(z)
        x = torch.zeros(1, 8, device=DEV)
        x[0, 0] = 1.0
        router = torch.zeros(E, 8, device=DEV)
        router[:, 0] = torch.tensor(z)
        ids, w = torch.empty(1, top, dtype=torch.int32, device=DEV), torch.empty(1, top, device=DEV)
        ops.moe_route(x, router, top, ids, w, scoring="softmax", groups=groups, groups_kept=kept,
                      correction=torch.tensor(corr, device=DEV), norm_eps=1e-20)
        return ids.cpu().tolist()[0], w.cpu()[0], torch.softmax(torch.tensor(z), dim=0)

    z = [2.0, 1.9, 0.0, 2.5, 2.2, -3.0]                       # three groups of two
    ids, w, s = route(z, [0.0] * 6, 2, 3, 2)
    assert ids == [3, 4]                                      # group 0 has the largest sum, groups 1 and 2 the largest entries
    assert torch.allclose(w, s[[3, 4]] / s[[3, 4]].sum(), atol=1e-6)
    ids, w, s = route(z, [0.0] * 6, 3, 3, 2)
    assert ids == [3, 4, 2]                                   # expert 2 (score 0) before experts 0 and 1 of the dropped group
    ids, w, s = route(z, [0.0, 0.0, 0.0, -1.0, 0.0, 0.9], 2, 3, 1)
    assert ids == [5, 4]                                      # the correction lifts expert 5 and with it group 2
    assert torch.allclose(w, s[[5, 4]] / s[[5, 4]].sum(), atol=1e-6)
    ids, w, s = route([0.0, 0.0, 0.0, 0.0], [-0.5, -0.6, -0.55, -0.7], 2, 2, 1)
    assert ids == [0, 1]                                      # all choice scores negative: expert 2 stays out of reach
    assert torch.allclose(w, torch.tensor([0.5, 0.5]), atol=1e-6)


@pytest.mark.parametrize("E,ident,ff,shared,top", [(6, 2, 24, 40, 3), (3, 1, 7, 0, 4), (4, 0, 10, 3, 2), (2, 3, 16, 8, 5),
                                                   (14, 2, 1024, 2048, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_identity_experts_and_the_shared_experts_sigmoid(E, ident, ff, shared, top, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(ff + ident)
    T, width = 11, (37 if ff == 7 else 40 if ff < 1024 else 4096)      # rows of 16-byte pieces and not
    n = E * ff + shared
    gu = torch.randn(T, 2 * n, generator=g).to(dtype)
    ids = torch.stack([torch.randperm(E + ident, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, top, generator=g) + 0.1
    logits = torch.randn(T, E + ident + 1, generator=g)
    sl = logits[:, E + ident] if shared else None
    act_ref = torch.empty(T, n, dtype=dtype)
    ref.moe_silu_gate_scale(gu, act_ref, ids, w, E, ff, shared, shared_logit=sl)
    act = torch.empty(T, n, dtype=dtype, device=DEV)
    ops.moe_silu_gate_scale(gu.to(DEV), act, ids.to(DEV), w.to(DEV), E, ff, shared,
                            shared_logit=logits.to(DEV)[:, E + ident] if shared else None)
    close(act, act_ref, 1e-5 if dtype == torch.float32 else 1e-2, "act")
    y, x = torch.randn(T, width, generator=g).to(dtype), torch.randn(T, width, generator=g).to(dtype)
    y_ref, y_gpu = y.clone(), y.clone().to(DEV)
    ref.moe_identity_add(y_ref, x, ids, w, E)
    ops.moe_identity_add(y_gpu, x.to(DEV), ids.to(DEV), w.to(DEV), E)
    close(y_gpu, y_ref, 1e-6 if dtype == torch.float32 else 1e-2, "identity")


@pytest.mark.parametrize("E,ident,ff,shared,top,width", [(6, 2, 24, 40, 3, 64), (3, 1, 7, 0, 4, 40), (4, 0, 10, 3, 2, 36),
                                                         (2, 3, 16, 8, 5, 128), (14, 2, 64, 128, 4, 512), (5, 1, 32, 8, 2, 72)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_experts_read_chosen_only(E, ident, ff, shared, top, width, dtype):
    """The few-token path against the plain double, and against the path that runs every expert: the same
    function of the same choices, the identity experts' share and the shared expert's sigmoid included."""
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(ff + ident + width)
    T = 5
    n = E * ff + shared
    x = torch.randn(T, width + 8, generator=g).to(dtype)[:, 8:]
    w_gu = (torch.randn(2 * n, width, generator=g) * width ** -0.5).to(dtype)
    w_down = (torch.randn(width, n, generator=g) * ff ** -0.5).to(dtype)
    ids = torch.stack([torch.randperm(E + ident, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if ident:
        ids[0, 0] = E + ident - 1                  # an identity expert in a fixed place too
        ids[0, 1:] = torch.arange(top - 1)
    w = torch.rand(T, top, generator=g) + 0.1
    logits = torch.randn(T, E + ident + 1, generator=g)
    sl = logits[:, E + ident] if shared else None
    act_ref = torch.empty(T, top * ff + shared, dtype=dtype)
    ref.moe_gate_up_chosen(x, w_gu, ids, w, act_ref, E, ff, shared, shared_logit=sl)
    act = torch.full((T, top * ff + shared), float("nan"), dtype=dtype, device=DEV)
    xd, idd, wd = x.to(DEV)[:, :], ids.to(DEV), w.to(DEV)
    xd = torch.cat([torch.zeros(T, 8, dtype=dtype, device=DEV), xd], dim=1)[:, 8:]       # rows wider than the width
    sld = logits.to(DEV)[:, E + ident] if shared else None
    ops.moe_gate_up_chosen(xd, w_gu.to(DEV), idd, wd, act, E, ff, shared, shared_logit=sld)
    close(act, act_ref, 2e-5 if dtype == torch.float32 else 1.5e-2, "act")
    out_ref = torch.empty(T, width, dtype=dtype)
    ref.moe_down_gated_chosen(act_ref, w_down, ids, w, x, out_ref, E, ff, shared)
    out = torch.empty(T, width, dtype=dtype, device=DEV)
    ops.moe_down_gated_chosen(act_ref.to(DEV), w_down.to(DEV), idd, wd, xd, out, E, ff, shared)
    close(out, out_ref, 2e-5 if dtype == torch.float32 else 1.5e-2, "out")
    # every expert through the products, the others' activations zero: the same sum
    gu = torch.empty(T, 2 * n, dtype=dtype, device=DEV)
    ops.linear(xd, w_gu.to(DEV), gu)
    full = torch.empty(T, n, dtype=dtype, device=DEV)
    ops.moe_silu_gate_scale(gu, full, idd, wd, E, ff, shared, shared_logit=sld)
    dense = torch.empty(T, width, dtype=dtype, device=DEV)
    ops.linear(full, w_down.to(DEV), dense)
    ops.moe_identity_add(dense, xd, idd, wd, E)
    close(out, dense.cpu(), 5e-5 if dtype == torch.float32 else 3e-2, "against every expert")


@pytest.mark.parametrize("H,N,K", [(3, 24, 48), (8, 48, 96), (5, 8, 40), (2, 128, 576), (1, 7, 19)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_products_with_one_gate_a_head(H, N, K, dtype):
    ops, ref = kernels.current(), KernelDouble()
    g = torch.Generator().manual_seed(N + K)
    T = 23
    x = torch.randn(T, H * K + 8, generator=g).to(dtype)
    weight = (torch.randn(H, N, K, generator=g) * K ** -0.5).to(dtype)
    gate = torch.randn(T, H + 3, generator=g).to(dtype)
    out_ref, out = torch.empty(T, H * N, dtype=dtype), torch.empty(T, H * N, dtype=dtype, device=DEV)
    ref.head_linear(x[:, :H * K], K, weight, out_ref, N, gate=gate[:, :H], gate_per_head=True)
    ops.head_linear(x.to(DEV)[:, :H * K], K, weight.to(DEV), out, N, gate=gate.to(DEV)[:, :H], gate_per_head=True)
    close(out, out_ref, 2e-5 if dtype == torch.float32 else 1.5e-2, "head_linear")
