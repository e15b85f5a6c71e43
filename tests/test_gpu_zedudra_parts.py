"""Each mechanism of Zedudra alone, the engine's kernels against the plain functions: norms in groups
(alone, with the residual add, as the pair around a residual add), the input convolution with its kept
rows (any mix of requests, slots used again, padding, one by one against a prompt), attention over a
window and kept first positions with the keys as values and a gate per head (scattered pages, far keys,
page borders, keys just inside and just outside the window and the kept positions, prompts and single
tokens), the xIELU activation, the router and the clamped experts."""
import numpy as np
import pytest
import torch

from plain import zedudra_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 2e-6, torch.bfloat16: 1e-2}


def ops_for(dtype):
    from minivllm_amd.kernels.ops import Ops
    return Ops(dtype)


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def step_ints(q_lens, slots, pad_rows=0, pad_seqs=0):
    seq = [s for s, n in enumerate(q_lens) for _ in range(n)] + [-1] * pad_rows
    cu = np.concatenate([[0], np.cumsum(q_lens)]).tolist()
    cu += [cu[-1]] * pad_seqs
    return i32(seq), i32(cu), i32(list(slots) + [0] * pad_seqs)


def close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= tol, f"{what}: relative error {err:.3e} exceeds {tol:.1e}"


# ---------------------------------------------------------------------------------------
# norms in groups
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h, groups", [(64, 4), (50, 5), (256, 1), (32, 16), (48, 2), (1000, 8), (30, 30), (4096, 2)])
def test_group_norm_rows(dtype, h, groups):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(h + groups)
    n, eps = 7, 3e-6
    resid = (3 * torch.randn(n, h, generator=g)).to(DEV)
    resid[:, : h // groups] *= 20                      # one group much larger than the rest: a norm over the whole row would show
    delta = torch.randn(n, h, generator=g).to(dtype).to(DEV)
    w = (1 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16).to(DEV)
    want_sum = resid.double() + delta.double()
    out = torch.empty(n, h, dtype=dtype, device=DEV)
    r = resid.clone()
    ops.group_norm(w, eps, groups, out, resid=r, delta=delta)
    close(r, want_sum, 1e-6, "the sum goes back to the residual")
    close(out, plain.grouped_rms_norm(want_sum.cpu(), w.double().cpu(), groups, eps), TOL[dtype], "add + norm")
    # some rows only (a negative row gives zeros), nothing written back
    rows = i32([5, -1, 0])
    r2, out2 = resid.clone(), torch.full((3, h), 7.0, dtype=dtype, device=DEV)
    ops.group_norm(w, eps, groups, out2, resid=r2, delta=delta, rows=rows)
    assert torch.equal(r2, resid) and float(out2[1].abs().max()) == 0
    close(out2[[0, 2]], plain.grouped_rms_norm(want_sum.cpu()[[5, 0]], w.double().cpu(), groups, eps), TOL[dtype], "chosen rows")
    # activation rows as they are, strided
    wide = torch.randn(n, h + 8, generator=g).to(dtype).to(DEV)
    out3 = torch.empty(n, h, dtype=dtype, device=DEV)
    ops.group_norm(w, eps, groups, out3, x=wide[:, :h])
    close(out3, plain.grouped_rms_norm(wide[:, :h].double().cpu(), w.double().cpu(), groups, eps), TOL[dtype], "plain rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h, groups, taps", [(64, 4, 3), (50, 5, 2), (256, 1, 4), (32, 16, 1), (48, 2, 0), (4096, 4, 4), (8192, 2, 3),
                                             (1024, 128, 2), (2056, 1, 1), (3072, 3, 5), (704, 88, 3), (8200, 1, 2)])
def test_norm_add_norm_in_groups_and_the_convolution_riding_along(dtype, h, groups, taps):
    """Rows the vector kernel takes (a multiple of eight columns in groups of a multiple of eight, up to 8,192, at most
    four taps given tap by tap) and rows it leaves to the general one; both against the plain norm, and the convolution
    that rides along against the separate kernel bit for bit."""
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(h)
    n = 5
    y = torch.randn(n, h, generator=g).to(dtype).to(DEV)
    resid = (2 * torch.randn(n, h, generator=g)).to(DEV)
    wa = (1 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16).to(DEV)
    wb = (1 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16).to(DEV)
    v = resid.double().cpu() + plain.grouped_rms_norm(y.double().cpu(), wa.double().cpu(), groups, 1e-5)
    normed = plain.grouped_rms_norm(v, wb.double().cpu(), groups, 2e-6)
    r, out = resid.clone(), torch.empty(n, h, dtype=dtype, device=DEV)
    ops.group_norm_add_norm(y, (wa, 1e-5), r, (wb, 2e-6), out, groups)
    close(r, v, 1e-6, "the residual after the add")
    close(out, normed, TOL[dtype], "the second norm")
    r2 = resid.clone()
    ops.group_norm_add_norm(y, (wa, 1e-5), r2, None, None, groups)
    assert torch.equal(r2, r)
    if taps == 0:
        return
    # steps of single tokens: rows of requests in slots 3, 0, 2 and two padding rows; the convolution as the separate kernel does it
    cw = (0.5 * torch.randn(h, taps, generator=g)).to(torch.bfloat16).to(DEV)
    state = torch.randn(4, max(taps - 1, 1), h, generator=g).to(dtype).to(DEV)[:, :taps - 1].contiguous() if taps > 1 else None
    tsq, cu, slots = i32([0, -1, 1, 2, -1]), i32([0, 1, 2, 3]), i32([3, 0, 2])
    cwt = cw.t().contiguous()
    real = [0, 2, 3]
    for by_tap in (False, True):
        s1 = state.clone() if state is not None else None
        r3, out3 = resid.clone(), torch.empty(n, h, dtype=dtype, device=DEV)
        ops.group_norm_add_norm(y, (wa, 1e-5), r3, (wb, 2e-6), out3, groups,
                                conv=(cw, s1, tsq, slots, cwt) if by_tap else (cw, s1, tsq, slots))
        close(r3, v, 1e-6, "the residual after the add, with the convolution riding along")
        # the same through the separate kernels on the three real rows
        s2 = state.clone() if state is not None else None
        mixed = torch.empty(3, h, dtype=dtype, device=DEV)
        ops.input_conv(out[real].contiguous(), cw, s2, i32([0, 1, 2]), cu, slots, 3, mixed, taps_t=cwt if by_tap else None)
        # (taps not given tap by tap go through the general kernel, whose norm sums in another order than the vector
        # kernel that made ``out``: equal within rounding there, bit for bit otherwise)
        exact = by_tap and taps <= 4          # the vector kernel takes up to four taps
        if exact:
            assert torch.equal(out3[real], mixed)
        else:
            close(out3[real], mixed, TOL[dtype], "the convolution riding along, general kernel")
        assert float(out3[[1, 4]].abs().max()) == 0
        if state is not None:
            if exact:
                assert torch.equal(s1, s2)
            else:
                close(s1, s2, TOL[dtype], "the kept rows, general kernel")
            assert torch.equal(s1[1], state[1])      # slot 1 belongs to nobody in the step


# ---------------------------------------------------------------------------------------
# input convolution
# ---------------------------------------------------------------------------------------
def conv_reference(h, taps, before):
    return plain.input_conv(h.double().cpu(), taps.double().cpu(), None if before is None else before.double().cpu())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("by_tap", [False, True])
@pytest.mark.parametrize("width, taps", [(64, 3), (50, 2), (256, 4), (30, 1), (40, 7), (4096, 4), (1032, 16)])
def test_input_convolution_mixed_step(dtype, width, taps, by_tap):
    """Three requests in one step (a long portion, a portion shorter than the taps reach back, a single token) in slots
    2, 0, 3 with non-zero kept rows, padding rows and a padding sequence; then a second step on what the first left."""
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(width * taps)
    cw = (0.5 * torch.randn(width, taps, generator=g)).to(torch.bfloat16).to(DEV)
    state = torch.randn(5, max(taps - 1, 1), width, generator=g).to(dtype).to(DEV)[:, :taps - 1].contiguous() if taps > 1 else None
    before = state.clone() if state is not None else None
    for q_lens in ([9, 2, 1], [1, 5, 3]):
        n = sum(q_lens)
        h = torch.randn(n + 2, width, generator=g).to(dtype).to(DEV)
        tsq, cu, slots = step_ints(q_lens, [2, 0, 3], pad_rows=2, pad_seqs=1)
        out = torch.full((n + 2, width), 5.0, dtype=dtype, device=DEV)
        ops.input_conv(h, cw, state, tsq, cu, slots, 4, out, taps_t=cw.t().contiguous() if by_tap else None)
        p = 0
        for s, ql in enumerate(q_lens):
            slot = [2, 0, 3][s]
            want, kept = conv_reference(h[p:p + ql], cw, None if state is None else before[slot])
            close(out[p:p + ql], want, TOL[dtype], f"request {s}")
            if state is not None:
                assert torch.equal(state[slot].double().cpu(), kept), f"kept rows of request {s}"
            p += ql
        assert float(out[n:].abs().max()) == 0
        if state is not None:
            assert torch.equal(state[1], before[1]) and torch.equal(state[4], before[4])     # slots of nobody
            before = state.clone()


@pytest.mark.parametrize("dtype", DTYPES)
def test_input_convolution_in_portions_is_the_whole_bit_for_bit(dtype):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(4)
    width, taps, n = 72, 4, 60
    cw = (0.5 * torch.randn(width, taps, generator=g)).to(torch.bfloat16).to(DEV)
    h = torch.randn(n, width, generator=g).to(dtype).to(DEV)

    def run(sizes, slot):
        state = torch.full((3, taps - 1, width), 9.0, dtype=dtype, device=DEV)
        state[slot] = 0                                    # what the executor does for a request that starts
        rows, p = [], 0
        for k in sizes:
            tsq, cu, slots = step_ints([k], [slot])
            out = torch.empty(k, width, dtype=dtype, device=DEV)
            ops.input_conv(h[p:p + k].contiguous(), cw, state, tsq, cu, slots, 1, out)
            rows.append(out)
            p += k
        assert p == n
        return torch.cat(rows)

    whole = run([n], 0)
    close(whole, conv_reference(h, cw, None)[0], TOL[dtype], "whole")
    for sizes in ([1] * n, [2] * 30, [3, 1, 2, 50, 4], [59, 1]):
        assert torch.equal(run(sizes, 2), whole), f"portions {sizes[:5]}"


# ---------------------------------------------------------------------------------------
# attention over a window and kept first positions
# ---------------------------------------------------------------------------------------
class AttentionCase:
    """One request of ``n`` tokens: packed rows [q | k | gates] as the projection leaves them, pages scattered over a
    pool whose other pages hold NaN."""

    def __init__(self, H, G, D, rot, base, n, page, seed, dtype, gain=1.0):
        self.H, self.G, self.D, self.rot, self.base, self.n, self.page, self.dtype = H, G, D, rot, base, n, page, dtype
        g = torch.Generator().manual_seed(seed)
        self.width = H * D + G * D + H
        self.width += (-self.width) % 8
        self.packed = (gain * torch.randn(n, self.width, generator=g)).to(dtype)
        self.packed[:, H * D + G * D:] /= gain
        n_pages = -(-n // page)
        pool = 2 * n_pages + 3
        self.table = torch.randperm(pool, generator=g)[:n_pages].tolist()
        self.k_pages = torch.full((pool, G, page, D), float("nan"), dtype=dtype, device=DEV)
        self.v_pages = torch.full((pool, G, D, page), float("nan"), dtype=dtype, device=DEV)
        self.ops = ops_for(dtype)
        self.table_dev = None
        if rot:
            from minivllm_amd.parts.rope import inverse_frequencies
            self.rope = self.ops.rope_table(inverse_frequencies(rot, base).to(DEV), n + 8)
        else:
            self.rope = None

    def want(self, window, first, scale):
        """float64 [n, H * D] by the plain functions (the values are the keys before rotation)."""
        H, G, D, n = self.H, self.G, self.D, self.n
        p = self.packed.double()
        pos = torch.arange(n)
        rnd = (lambda t: t.to(self.dtype).double())
        q = rnd(plain.rotate_pairs(p[:, :H * D].reshape(n, H, D), pos, self.rot, self.base))
        k0 = p[:, H * D:H * D + G * D].reshape(n, G, D)
        k = rnd(plain.rotate_pairs(k0, pos, self.rot, self.base))
        gate = torch.sigmoid(p[:, H * D + G * D:H * D + G * D + H])
        allowed = plain.visibility(0, n, window, first)
        out = torch.zeros(n, H, D, dtype=torch.float64)
        for hd in range(H):
            s = (q[:, hd] @ k[:, hd // (H // G)].T) * scale
            s = torch.where(allowed, s, torch.full_like(s, float("-inf")))
            out[:, hd] = torch.softmax(s, -1) @ k0[:, hd // (H // G)]
        return (out * gate[:, :, None]).reshape(n, H * D)

    def run(self, steps, window, first, scale, drop_pages=False, variant=None):
        """Feeds the request in steps of the given sizes; returns [n, H * D]. ``drop_pages``: a page that neither the
        window nor the kept positions need any more is taken out of the block table (and filled with NaN) before a step.
        ``variant``: (column tiles a wave, key groups a workgroup) of the MFMA prompt kernel instead of the launch rule's."""
        from minivllm_amd.engine.step import AttentionPlan
        from minivllm_amd.parts.base import Workspace
        H, G, D, page = self.H, self.G, self.D, self.page
        ws = Workspace(torch.device(DEV))
        rows, p = [], 0
        table = list(self.table)
        for k in steps:
            if drop_pages:
                for i in range(len(table)):
                    if i >= -(-first // page) and (i + 1) * page - 1 < p - (window - 1) and table[i] >= 0:
                        self.k_pages[table[i]] = float("nan")
                        self.v_pages[table[i]] = float("nan")
                        table[i] = -1
            packed = self.packed[p:p + k].to(DEV).contiguous()
            positions, tsq = i32(range(p, p + k)), i32([0] * k)
            bt = i32(table).view(1, -1)
            held = H * D + G * D
            self.ops.qk_norm_rope_store(packed, H, G, D, positions, tsq, None, None, 1e-6, self.rope, True, self.k_pages,
                                        self.v_pages, bt, page, value_from_key=True, extra_columns=self.width - held)
            out = torch.empty(k, H * D, dtype=self.dtype, device=DEV)
            plan = AttentionPlan(decode_only=(k == 1), max_q_len=k, max_context_len=p + k, n_seqs=1, q_lens=[k],
                                 cu_seqlens=i32([0, k]), workspace=ws, prefill_variant=variant if k > 1 else None)
            self.ops.attention(packed[:, :H * D], out, self.k_pages, self.v_pages, bt, page, positions, tsq, H, G, D, scale,
                               window - 1, plan=plan, keep_first=first, gate=packed[:, held:held + H])
            rows.append(out)
            p += k
        assert p == self.n
        return torch.cat(rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, rot, window, first, page", [
    (4, 2, 16, 8, 12, 5, 16), (3, 3, 10, 10, 7, 0, 8), (4, 1, 64, 32, 40, 17, 16), (2, 2, 128, 64, 100, 64, 16),
    (1, 1, 12, 0, 4, 30, 4), (2, 1, 20, 6, 1, 6, 16), (8, 2, 64, 64, 33, 16, 16), (6, 2, 8, 8, 500, 3, 8)])
def test_attention_whole_in_portions_and_token_by_token(dtype, H, G, D, rot, window, first, page):
    case = AttentionCase(H, G, D, rot, 1000.0, 150, page, seed=H * D + window, dtype=dtype, gain=1.5)
    scale = D ** -0.5
    want = case.want(window, first, scale)
    tol = 3e-5 if dtype == torch.float32 else 2.5e-2
    close(case.run([150], window, first, scale), want, tol, "whole")
    close(case.run([7, 5, 3, 2, 11, 2, 17, 2, 4, 60, 1, 1, 35], window, first, scale, drop_pages=True), want, tol, "portions")
    close(case.run([110] + [1] * 40, window, first, scale, drop_pages=True), want, tol, "the last 40 one by one")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("single", [False, True])
def test_one_key_that_stands_out_is_seen_exactly_where_the_mask_says(dtype, single):
    """The query at the last position points at one key whose score stands out by far; the output is that key's value
    when the key is visible and nothing like it when it is not. Keys just inside and just outside the window, the last
    kept position and the first one behind them, at page borders, hundreds of positions back; in a prompt and as a
    single token."""
    H, G, D, page, window, first, n = 2, 1, 32, 16, 48, 17, 400
    for target, seen in ((n - 1, True), (n - window, True), (n - window - 1, False), (first - 1, True), (first, False),
                         (0, True), (15, True), (16, True), (17, False), (n - 49, False), (n - 1 - 31, True), (n - 1 - 32, True)):
        case = AttentionCase(H, G, D, 0, 1.0, n, page, seed=target + 1, dtype=dtype, gain=0.3)
        direction = torch.zeros(D)
        direction[target % D] = 1.0
        case.packed[target, H * D:H * D + D] = (6.0 * direction).to(dtype)                    # the key (and the value)
        case.packed[n - 1, :H * D] = (6.0 * direction).repeat(H).to(dtype)                    # both heads' queries
        case.packed[:, H * D + G * D:H * D + G * D + H] = 8.0                                 # gates open
        got = case.run([n - 1, 1] if single else [n], window, first, 1.0)[n - 1].double().cpu().view(H, D)
        hit = got[:, target % D]
        if seen:
            assert float(hit.min()) > 5.5, f"key {target} should be seen: {hit.tolist()}"
        else:
            assert float(hit.abs().max()) < 1.0, f"key {target} should not be seen: {hit.tolist()}"
        close(got.view(1, -1), case.want(window, first, 1.0)[n - 1:n], 3e-5 if dtype == torch.float32 else 2.5e-2, f"key {target}")


@pytest.mark.parametrize("nt, kw", [(1, 1), (1, 2), (2, 1), (2, 2)])
@pytest.mark.parametrize("H, G, window, first", [(4, 2, 36, 13), (3, 1, 50, 33), (2, 2, 24, 45)])
def test_kept_positions_in_every_variant_of_the_prompt_kernel(nt, kw, H, G, window, first):
    """Every query points at one kept position, so its output is that key's value wherever it lies. A unit of queries
    whose first windows still reach the block of the kept positions and whose last ones do not must look at that block
    for all of them, with four waves and with eight (two groups that take the blocks of keys in turn)."""
    dtype, D, page, n = torch.bfloat16, 64, 16, 300
    case = AttentionCase(H, G, D, 0, 1.0, n, page, seed=nt * 10 + kw + window, dtype=dtype, gain=0.3)
    direction = torch.zeros(D)
    direction[3] = 1.0
    target = first - 1
    case.packed[target, H * D:H * D + G * D] = (6.0 * direction).repeat(G).to(dtype)
    case.packed[:, :H * D] = (6.0 * direction).repeat(H).to(dtype)
    case.packed[:, H * D + G * D:H * D + G * D + H] = 8.0
    want = case.want(window, first, 1.0)
    for steps in ([n], [5, 128, 64, 3, 100], [61, 2, 237]):
        got = case.run(steps, window, first, 1.0, drop_pages=True, variant=(nt, kw))
        hit = got.double().cpu().view(n, H, D)[target:, :, 3]
        assert float(hit.min()) > 5.0, f"steps {steps}: the kept key is lost at {int((hit.min(1).values < 5.0).nonzero()[0]) + target}"
        close(got, want, 2.5e-2, f"steps {steps}")


# ---------------------------------------------------------------------------------------
# feed-forwards
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_xielu(dtype):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(1)
    x = (3 * torch.randn(9, 70, generator=g)).to(dtype).to(DEV)
    x[0, :4] = torch.tensor([0.0, -0.0, 1e-3, -1e-3]).to(dtype)
    p, q = torch.tensor(0.37, dtype=torch.float64), torch.tensor(-0.8, dtype=torch.float64)
    out = torch.empty_like(x)
    ops.xielu(x, float(plain.softplus(p)), 0.5 + float(plain.softplus(q)), out)
    close(out, plain.xielu(x.double().cpu(), p, q), TOL[dtype], "xielu")
    wide = torch.zeros(9, 80, dtype=dtype, device=DEV)
    wide[:, :70] = x
    ops.xielu(wide[:, :70], float(plain.softplus(p)), 0.5 + float(plain.softplus(q)), wide[:, :70])      # in place, strided
    assert torch.equal(wide[:, :70], out)
    # rows of a multiple of eight columns go eight columns a thread; the same numbers as one column a thread
    x8 = (3 * torch.randn(33, 264, generator=g)).to(dtype).to(DEV)
    x8[1, 5:9] = torch.tensor([0.0, -0.0, 1e-3, -1e-3]).to(dtype)
    out8 = torch.empty_like(x8)
    ops.xielu(x8, float(plain.softplus(p)), 0.5 + float(plain.softplus(q)), out8)
    close(out8, plain.xielu(x8.double().cpu(), p, q), TOL[dtype], "xielu, eight columns a thread")
    odd = torch.empty(33, 263, dtype=dtype, device=DEV)
    ops.xielu(x8[:, :263], float(plain.softplus(p)), 0.5 + float(plain.softplus(q)), odd)
    assert torch.equal(odd, out8[:, :263])


@pytest.mark.parametrize("E, groups, keep, top", [(16, 4, 2, 3), (8, 4, 2, 4), (6, 1, 1, 2), (5, 5, 3, 2), (3, 1, 1, 3),
                                                  (64, 8, 3, 6), (12, 2, 1, 6), (9, 3, 3, 4)])
def test_router_against_the_plain_choice(E, groups, keep, top):
    ops = ops_for(torch.float32)
    g = torch.Generator().manual_seed(E * top)
    n = 200
    z = 2 * torch.randn(n, E, generator=g)
    dense = torch.full((n, E), 5.0, device=DEV)
    ids = torch.empty(n, top, dtype=torch.int32, device=DEV)
    weights = torch.empty(n, top, device=DEV)
    ops.moe_route(z.to(DEV), None, groups, keep, top, 1e-20, dense, ids, weights, scoring="sigmoid", group_worth="top2",
                  normalize=False)
    want_ids, want_w = plain.route(z.double(), groups, keep, top)
    assert torch.equal(ids.cpu().long(), want_ids), "the chosen experts, in the order of choice"
    close(weights, want_w, 1e-6, "the weights are the scores themselves")
    full = torch.zeros(n, E, dtype=torch.float64).scatter_(1, want_ids, want_w)
    close(dense, full, 1e-6, "dense weights")
    # the other options stay what they were: softmax scores, a group's largest choice, weights that sum to one
    ops.moe_route(z.to(DEV), None, groups, keep, top, 1e-20, dense, ids, weights)
    assert torch.allclose(weights.sum(-1).cpu(), torch.ones(n), atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hid, F, E, groups, keep, top, limit", [(64, 24, 8, 4, 2, 3, 1.5), (50, 22, 6, 1, 1, 2, 0.7),
                                                                (32, 16, 3, 1, 1, 3, 3.0), (48, 20, 5, 5, 3, 2, 1.2)])
def test_routed_clamped_experts_against_the_plain_mixture(dtype, hid, F, E, groups, keep, top, limit):
    from minivllm_amd.parts.base import Runtime, Workspace
    from minivllm_amd.parts.moe import RoutedExperts, RoutedExpertsSpec
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(hid + E)
    n = 37
    w = {"router": 3 * torch.randn(E, hid, generator=g) / hid ** 0.5}
    for e in range(E):
        w[f"gate.{e}"] = 2 * torch.randn(F, hid, generator=g) / hid ** 0.5      # many gates and ups beyond the limit
        w[f"up.{e}"] = 2 * torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"down.{e}"] = torch.randn(hid, F, generator=g) / F ** 0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    spec = RoutedExpertsSpec(hidden_size=hid, expert_size=F, num_experts=E, top=top, groups=groups, keep_groups=keep,
                             scoring="sigmoid", group_worth="top2", normalize=False, activation="clamped", limit=limit)
    rt = Runtime(device=torch.device(DEV), dtype=dtype, ops=ops, workspace=Workspace(torch.device(DEV)), max_positions=64)
    part = RoutedExperts(spec, {k: v.to(DEV) for k, v in w.items()}, rt)
    x = torch.randn(n, hid, generator=g).to(dtype)
    got = part.forward(x.to(DEV), None)
    names = {"mlp.router": w["router"].double()}
    for e in range(E):
        names.update({f"mlp.e{e}.gate": w[f"gate.{e}"].double(), f"mlp.e{e}.up": w[f"up.{e}"].double(),
                      f"mlp.e{e}.down": w[f"down.{e}"].double()})
    f = {"expert": {"ff": F, "limit": limit}, "router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}}
    want = plain.moe_ff(x.double(), names, "mlp.", f)
    close(got, want, 3e-5 if dtype == torch.float32 else 3e-2, "mixture")


@pytest.mark.parametrize("n, hid, F, E, groups, keep, top, limit", [(5, 64, 32, 8, 4, 2, 3, 1.5), (70, 96, 64, 6, 1, 1, 2, 0.7),
                                                                    (1, 128, 32, 16, 2, 1, 4, 2.0)])
def test_clamped_experts_over_the_chosen_pairs_only(n, hid, F, E, groups, keep, top, limit):
    """The path that computes only the chosen (token, expert) pairs (bfloat16, steps of few rows against large experts)
    with the clamped pair in its first product: against the plain mixture, and the kernels it ran are the grouped ones."""
    from minivllm_amd.parts.base import Runtime, Workspace
    from minivllm_amd.parts.moe import RoutedExperts, RoutedExpertsSpec
    dtype = torch.bfloat16
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(n + E)
    w = {"router": 3 * torch.randn(E, hid, generator=g) / hid ** 0.5}
    for e in range(E):
        w[f"gate.{e}"] = 2 * torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"up.{e}"] = 2 * torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"down.{e}"] = torch.randn(hid, F, generator=g) / F ** 0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    spec = RoutedExpertsSpec(hidden_size=hid, expert_size=F, num_experts=E, top=top, groups=groups, keep_groups=keep,
                             scoring="sigmoid", group_worth="top2", normalize=False, activation="clamped", limit=limit,
                             grouped=True, grouped_max_rows=1e9, grouped_min_weight=0)
    rt = Runtime(device=torch.device(DEV), dtype=dtype, ops=ops, workspace=Workspace(torch.device(DEV)), max_positions=64)
    part = RoutedExperts(spec, {k: v.to(DEV) for k, v in w.items()}, rt)
    x = torch.randn(n, hid, generator=g).to(dtype)
    ledger, ops.ledger = ops.ledger, []
    try:
        got = part.forward(x.to(DEV), None).clone()
        seen = [line[0] for line in ops.ledger]
    finally:
        ops.ledger = ledger
    assert "mv_moe_grouped" in seen and "mv_moe_swiglu_scale" not in seen, seen
    names = {"mlp.router": w["router"].double()}
    for e in range(E):
        names.update({f"mlp.e{e}.gate": w[f"gate.{e}"].double(), f"mlp.e{e}.up": w[f"up.{e}"].double(),
                      f"mlp.e{e}.down": w[f"down.{e}"].double()})
    f = {"expert": {"ff": F, "limit": limit}, "router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}}
    close(got, plain.moe_ff(x.double(), names, "mlp.", f), 3e-2, "mixture over the chosen pairs")


@pytest.mark.parametrize("dtype", DTYPES)
def test_dense_feed_forward_against_the_plain_one(dtype):
    from minivllm_amd.parts.base import Runtime, Workspace
    from minivllm_amd.parts.mlp import XIELUFeedForward, XIELUSpec
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(8)
    hid, ff, n = 56, 90, 21
    w = {"up": (2 * torch.randn(ff, hid, generator=g) / hid ** 0.5).to(torch.bfloat16),
         "down": (torch.randn(hid, ff, generator=g) / ff ** 0.5).to(torch.bfloat16),
         "act": torch.tensor([0.6, -1.1]).to(torch.bfloat16)}
    rt = Runtime(device=torch.device(DEV), dtype=dtype, ops=ops, workspace=Workspace(torch.device(DEV)), max_positions=64)
    part = XIELUFeedForward(XIELUSpec(hidden_size=hid, intermediate_size=ff), {k: v.to(DEV) for k, v in w.items()}, rt)
    x = torch.randn(n, hid, generator=g).to(dtype)
    got = part.forward(x.to(DEV), None)
    if not isinstance(got, torch.Tensor):
        got = got.materialize()
    want = plain.dense_ff(x.double(), {"mlp." + k: v.double() for k, v in w.items()}, "mlp.")
    close(got, want, 3e-5 if dtype == torch.float32 else 3e-2, "dense feed-forward")
