"""Each mechanism of Furanex alone, the engine's kernels and parts against the plain functions: the residual
streams' step (first read, write and read, last write and sum; the general and the vector kernel), grouped
attention with rotation first and the unit norm second, values of another size than keys and values blended
with another layer's (scattered pages, far keys, page borders, first tokens, prompts and single tokens),
attention over a latent with neighbour pairs and a gate per head, experts named by a table beside a shared
expert (all experts at once, the chosen pairs only)."""
import numpy as np
import pytest
import torch

from plain import furanex_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops_for(dtype):
    from minivllm_amd.kernels.ops import Ops
    return Ops(dtype)


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= tol, f"{what}: relative error {err:.3e} exceeds {tol:.1e}"


def runtime(dtype, max_positions=2048):
    from minivllm_amd.parts.base import Runtime, Workspace
    return Runtime(device=torch.device(DEV), dtype=dtype, ops=ops_for(dtype), workspace=Workspace(torch.device(DEV)),
                   max_positions=max_positions)


class Paged:
    """One request on scattered pages (every page nobody owns holds NaN) and the contexts of its steps."""

    def __init__(self, rt, need, n, page, seed, spare=5):
        self.rt, self.page = rt, page
        count = -(-n // page)
        g = torch.Generator().manual_seed(seed)
        self.table = torch.randperm(count + spare, generator=g)[:count].tolist()
        self.pages = {name: torch.full((count + spare,) + tuple(shape), float("nan"), dtype=rt.dtype, device=DEV)
                      for name, shape in need.page_shapes(page).items()}

    def ctx(self, start, k, token_ids=None):
        from minivllm_amd.engine.step import AttentionPlan, KVView, StepContext
        ctx = StepContext()
        ctx.n_tokens, ctx.n_seqs = k, 1
        ctx.positions, ctx.token_seq = i32(range(start, start + k)), i32([0] * k)
        ctx.cu_seqlens, ctx.context_lens, ctx.state_slots = i32([0, k]), i32([start + k]), i32([0])
        ctx.token_ids = i32(token_ids if token_ids is not None else [0] * k)
        ctx.q_lens, ctx.starts, ctx.page_size = [k], [start], self.page
        ctx._kv[0] = KVView(self.pages, i32(self.table).view(1, -1), self.page)
        ctx.attention_plan = AttentionPlan(decode_only=(k == 1), max_q_len=k, max_context_len=start + k, n_seqs=1, q_lens=[k],
                                           cu_seqlens=ctx.cu_seqlens, workspace=self.rt.workspace, kv_tokens=start + k)
        return ctx


# ---------------------------------------------------------------------------------------
# residual streams
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("S, W", [(4, 384), (3, 48), (2, 50), (1, 32), (5, 64), (8, 40), (4, 1024), (2, 4096), (3, 8200), (4, 8192)])
def test_stream_step(dtype, S, W):
    """The three shapes of the step against the plain read and write: widths and stream counts the vector kernel takes
    (a multiple of four columns up to 8,192, at most four streams) and those it leaves to the general one."""
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(S * 1000 + W)
    n, eps = 6, 2e-6
    emb = (3 * torch.randn(n, W, generator=g))
    w_in = [(1.0 / S + 0.2 * torch.randn(S, generator=g)) for _ in range(2)]
    w_out = [(1 + 0.3 * torch.randn(S, generator=g)) for _ in range(2)]
    w_mix = [(torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)) for _ in range(2)]
    norm_w = [(1 + 0.1 * torch.randn(W, generator=g)).to(torch.bfloat16) for _ in range(2)]
    wide = torch.randn(n, W + 8, generator=g).to(dtype)                  # the sublayer outputs, rows with a pitch of their own
    y = [wide[:, :W], torch.randn(n, W, generator=g).to(dtype)]
    tol = 2e-6 if dtype == torch.float32 else 1e-2
    # plain: all streams equal the embedding; read 0, write 0, read 1, write 1, sum
    xs = emb.double()[None].repeat(S, 1, 1)
    want_h0 = plain.rms_norm(plain.streams_read(xs, w_in[0].double()), norm_w[0].double(), eps)
    xs = plain.streams_write(xs, y[0].double(), w_mix[0].double(), w_out[0].double())
    lanes_1 = xs.clone()
    want_h1 = plain.rms_norm(plain.streams_read(xs, w_in[1].double()), norm_w[1].double(), eps)
    xs = plain.streams_write(xs, y[1].double(), w_mix[1].double(), w_out[1].double())
    want_total = xs.sum(0)
    # the engine: first read, write + read, write + sum
    lanes = torch.full((S, n, W), float("nan"), device=DEV)
    h = torch.empty(n, W, dtype=dtype, device=DEV)
    dev = lambda t: t.to(DEV).contiguous()
    ops.hyper_step(lanes, out=h, first=dev(emb), read=(dev(w_in[0]), dev(norm_w[0]), eps))
    close(h, want_h0, tol, "first read")
    close(lanes, emb.double()[None].repeat(S, 1, 1), 1e-7, "the streams start as the embedding")
    ops.hyper_step(lanes, out=h, write=(wide.to(DEV)[:, :W], dev(w_mix[0]), dev(w_out[0])), read=(dev(w_in[1]), dev(norm_w[1]), eps))
    close(lanes, lanes_1, 2e-6, "the streams after the first write")
    close(h, want_h1, tol, "second read")
    total = torch.full((n, W), float("nan"), device=DEV)
    ops.hyper_step(lanes, write=(dev(y[1]), dev(w_mix[1]), dev(w_out[1])), total=total)
    close(total, want_total, 2e-6, "sum of the streams after the last write")


# ---------------------------------------------------------------------------------------
# grouped attention: rotation, then the unit norm; values of their own size, blended with another layer's
# ---------------------------------------------------------------------------------------
STRETCH = {"factor": 3.0, "original": 64, "fast": 16.0, "slow": 2.0}


def attention_case(H, G, D, Dv, rot, width, seed, n, mixes):
    g = torch.Generator().manual_seed(seed)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": 6.0 / D}
    if rot:
        m["rot"] = {"dims": rot, "base": 700.0, "scaling": dict(STRETCH)}
    w = {"x.q": torch.randn(H * D, width, generator=g) / width ** 0.5, "x.k": torch.randn(G * D, width, generator=g) / width ** 0.5,
         "x.v": torch.randn(G * Dv, width, generator=g) / width ** 0.5, "x.o": torch.randn(width, H * Dv, generator=g) / (H * Dv) ** 0.5,
         "x.vmix": torch.tensor(0.37)}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    h = torch.randn(n, width, generator=g)
    first_values = 3.0 * torch.randn(n, G * Dv, generator=g) if mixes else None
    return m, w, h, first_values


def build_attention(rt, m, w, width, eps, mixes):
    from minivllm_amd.parts.attention import Attention, AttentionSpec
    from minivllm_amd.parts.rope import RotaryEmbedding, RotarySpec
    rot = m.get("rot")
    rope = None if not rot else RotarySpec(rotary_dim=rot["dims"], theta=rot["base"], stretch=tuple(
        rot["scaling"][k] for k in ("factor", "original", "fast", "slow")))
    spec = AttentionSpec(hidden_size=width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], scale=m["scale"],
                         qk_norm_eps=eps, position=rope, value_dim=m["vdim"], unit_norm_after_rotation=True,
                         value_mix="blend" if mixes else None, value_mix_key="first" if mixes else "")
    tensors = {k: w["x." + k].to(DEV) for k in ("q", "k", "v", "o")}
    if mixes:
        tensors["value_mix"] = w["x.vmix"].to(DEV)
    position = RotaryEmbedding(rope, {}, rt) if rope is not None else None
    return Attention(spec, tensors, rt, position=position), Attention.cache_need(spec)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, Dv, rot, width, page, mixes", [
    (4, 2, 16, 8, 12, 48, 16, True), (3, 3, 10, 14, 10, 50, 8, False), (6, 3, 64, 64, 64, 128, 16, True),
    (2, 1, 128, 128, 128, 64, 16, True), (2, 2, 8, 20, 4, 32, 4, True), (1, 1, 12, 12, 0, 40, 16, False),
    (4, 1, 64, 64, 32, 96, 16, True), (6, 2, 64, 32, 64, 64, 16, False), (2, 2, 256, 256, 256, 64, 16, True)])
def test_attention_whole_in_portions_and_token_by_token(dtype, H, G, D, Dv, rot, width, page, mixes):
    n, eps = 150, 1e-5
    m, w, h, first_values = attention_case(H, G, D, Dv, rot, width, seed=H * D + Dv, n=n, mixes=mixes)
    w64 = {k: v.double() for k, v in w.items()}
    hx = h.to(dtype)
    fv = None if first_values is None else first_values.to(dtype)
    want = plain.attention_mixer(hx.double(), w64, "x.", m, eps, first_values=None if fv is None else fv.double().view(n, G, Dv),
                                 mixes=mixes)[0]
    tol = 3e-5 if dtype == torch.float32 else 2.5e-2
    for what, steps in (("whole", [150]), ("portions", [7, 5, 3, 2, 11, 2, 17, 2, 4, 60, 1, 1, 35]), ("the last 40 one by one", [110] + [1] * 40)):
        rt = runtime(dtype)
        part, need = build_attention(rt, m, w, width, eps, mixes)
        paged = Paged(rt, need, n, page, seed=n + page)
        rows, p = [], 0
        for k in steps:
            ctx = paged.ctx(p, k)
            if mixes:
                ctx.carry["first"] = fv[p:p + k].to(DEV).contiguous()
            y = part.forward(hx[p:p + k].to(DEV).contiguous(), ctx, 0)
            rows.append((y if isinstance(y, torch.Tensor) else y.materialize()).clone())
            p += k
        close(torch.cat(rows), want, tol, what)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("single", [False, True])
@pytest.mark.parametrize("D, Dv", [(32, 24), (64, 64)])
def test_one_key_that_stands_out_is_found_wherever_it_lies(dtype, single, D, Dv):
    """The query at the last position points at one key; q and k are unit vectors, so the score of that key is
    scale * D and every other key's is small. The output is that key's value: at the first positions, at a page's last
    slot and the next page's first, hundreds of positions back, and the query's own. The query just in front of the key
    does not see it."""
    from minivllm_amd.engine.step import AttentionPlan
    from minivllm_amd.parts.base import KeepAll, KeyValueNeed, Workspace
    ops = ops_for(dtype)
    H, G, page, n = 2, 1, 16, 420
    ws = Workspace(torch.device(DEV))
    for target in (0, 1, 15, 16, 17, 31, 32, n - 401, n - 2, n - 1):
        g = torch.Generator().manual_seed(target + D)
        packed = 0.3 * torch.randn(n, H * D + G * D + G * Dv, generator=g)
        direction = torch.zeros(D)
        direction[target % D] = 1.0
        packed[target, H * D:H * D + D] = 6.0 * direction
        packed[n - 1, :H * D] = (6.0 * direction).repeat(H)
        if target > 0:
            packed[target - 1, :H * D] = (6.0 * direction).repeat(H)       # the query in front of the key asks for it too
        marker = torch.zeros(Dv)
        marker[target % Dv] = 5.0
        packed[target, H * D + G * D:] = marker
        packed = packed.to(dtype)
        paged = Paged(type("R", (), {"dtype": dtype, "workspace": ws})(), KeyValueNeed(KeepAll(), G, D, Dv), n, page, seed=target)
        bt = i32(paged.table).view(1, -1)
        outs, p = [], 0
        for k in ([n - 1, 1] if single else [n]):
            rows = packed[p:p + k].to(DEV).contiguous()
            pos, tsq = i32(range(p, p + k)), i32([0] * k)
            ops.qkv_rotate_norm_store(rows, H, G, D, Dv, pos, tsq, None, False, True, 1e-6, paged.pages["k"], paged.pages["v"], bt, page)
            out = torch.empty(k, H * Dv, dtype=dtype, device=DEV)
            plan = AttentionPlan(decode_only=(k == 1), max_q_len=k, max_context_len=p + k, n_seqs=1, q_lens=[k],
                                 cu_seqlens=i32([0, k]), workspace=ws)
            ops.attention(rows[:, :H * D], out, paged.pages["k"], paged.pages["v"], bt, page, pos, tsq, H, G, D, 1.0, None, plan=plan,
                          value_dim=Dv)
            outs.append(out)
            p += k
        got = torch.cat(outs).double().cpu().view(n, H, Dv)
        assert float(got[n - 1, :, target % Dv].min()) > 4.5, f"key {target} should be found: {got[n - 1, :, target % Dv].tolist()}"
        if target > 0:
            assert float(got[target - 1, :, target % Dv].abs().max()) < 1.0, f"key {target} lies behind the query at {target - 1}"


# ---------------------------------------------------------------------------------------
# attention over a latent: neighbour pairs, stretched frequencies, a gate per head
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, D, Dr, Dv, Q, R, width, page", [(3, 12, 4, 8, 24, 16, 48, 16), (5, 6, 2, 10, 14, 18, 50, 8),
                                                             (6, 24, 32, 40, 64, 128, 192, 16), (1, 20, 0, 6, 10, 12, 32, 4),
                                                             (16, 64, 64, 64, 96, 256, 128, 16), (2, 16, 16, 8, 32, 64, 64, 16)])
def test_latent_attention_whole_in_portions_and_token_by_token(dtype, H, D, Dr, Dv, Q, R, width, page):
    from minivllm_amd.parts.latent_attention import LatentAttention, LatentAttentionSpec
    from minivllm_amd.parts.rope import RotaryEmbedding, RotarySpec
    n, eps = 150, 1e-5
    g = torch.Generator().manual_seed(H * D + R)
    m = {"heads": H, "dim": D, "rot_dim": Dr, "vdim": Dv, "q_rank": Q, "kv_rank": R, "scale": 0.3}
    if Dr:
        m["rot"] = {"dims": Dr, "base": 300.0, "scaling": {"factor": 2.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    shapes = {"dq": (Q, width), "uq": (H * (D + Dr), Q), "dkv": (R + Dr, width), "uk": (H * D, R), "uv": (H * Dv, R), "g": (H, width),
              "o": (width, H * Dv)}
    w = {"x." + k: (2.0 if k == "uq" else 1.0) * torch.randn(s, generator=g) / s[1] ** 0.5 for k, s in shapes.items()}
    w["x.dq.norm"], w["x.dkv.norm"] = 1 + 0.1 * torch.randn(Q, generator=g), 1 + 0.1 * torch.randn(R, generator=g)
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    hx = torch.randn(n, width, generator=g).to(dtype)
    want = plain.latent_attention_mixer(hx.double(), {k: v.double() for k, v in w.items()}, "x.", m, eps)[0]
    rope = None if not Dr else RotarySpec(rotary_dim=Dr, theta=300.0, stretch=(2.0, 32, 8.0, 1.0))
    spec = LatentAttentionSpec(hidden_size=width, num_heads=H, plain_dim=D, rot_dim=Dr, value_dim=Dv, q_rank=Q, kv_rank=R, scale=0.3,
                               norm_eps=eps, output_gate=True, head_gate=True, rot_neighbours=True, position=rope)
    names = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "g": "g", "o": "o"}
    tol = 3e-5 if dtype == torch.float32 else 2.5e-2
    for what, steps in (("whole", [150]), ("portions", [7, 5, 3, 2, 11, 2, 17, 2, 4, 60, 1, 1, 35]), ("the last 40 one by one", [110] + [1] * 40)):
        rt = runtime(dtype)
        part = LatentAttention(spec, {k: w["x." + v].to(DEV) for k, v in names.items()}, rt,
                               position=RotaryEmbedding(rope, {}, rt) if rope is not None else None)
        paged = Paged(rt, LatentAttention.cache_need(spec), n, page, seed=n + page)
        rows, p = [], 0
        for k in steps:
            y = part.forward(hx[p:p + k].to(DEV).contiguous(), paged.ctx(p, k), 0)
            rows.append((y if isinstance(y, torch.Tensor) else y.materialize()).clone())
            p += k
        close(torch.cat(rows), want, tol, what)


# ---------------------------------------------------------------------------------------
# experts named by a table, beside a shared expert
# ---------------------------------------------------------------------------------------
def mixture_case(hid, F, E, top, FS, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for e in range(E):
        w[f"m.e{e}.gate"] = torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"m.e{e}.up"] = torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"m.e{e}.down"] = torch.randn(hid, F, generator=g) / F ** 0.5
    if FS:
        w["m.shared.gate"] = torch.randn(FS, hid, generator=g) / hid ** 0.5
        w["m.shared.up"] = torch.randn(FS, hid, generator=g) / hid ** 0.5
        w["m.shared.down"] = torch.randn(hid, FS, generator=g) / FS ** 0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    w["m.table"] = torch.rand((vocab, E), generator=g).argsort(dim=1)[:, :top].to(torch.int32).contiguous()
    f = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": top}}
    if FS:
        f["shared"] = {"ff": FS}
    return w, f


def build_mixture(rt, w, hid, F, E, top, FS, vocab, **options):
    from minivllm_amd.parts.moe import RoutedExperts, RoutedExpertsSpec
    spec = RoutedExpertsSpec(hidden_size=hid, expert_size=F, num_experts=E, top=top, router="table", table_rows=vocab, shared_size=FS,
                             **options)
    tensors = {"table": w["m.table"].to(DEV)}
    for e in range(E):
        for k in ("gate", "up", "down"):
            tensors[f"{k}.{e}"] = w[f"m.e{e}.{k}"].to(DEV)
    if FS:
        for k in ("gate", "up", "down"):
            tensors[f"shared.{k}"] = w[f"m.shared.{k}"].to(DEV)
    return RoutedExperts(spec, tensors, rt)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hid, F, E, top, FS", [(48, 24, 5, 2, 40), (50, 22, 3, 1, 0), (256, 64, 10, 1, 128), (40, 10, 4, 4, 26), (64, 16, 1, 1, 8)])
def test_table_mixture_against_the_plain_one(dtype, hid, F, E, top, FS):
    """A row's experts follow its token id alone: the same ids in another order, beside other rows, give the same rows."""
    vocab, n = 37, 60
    w, f = mixture_case(hid, F, E, top, FS, vocab, seed=hid + E)
    rt = runtime(dtype)
    part = build_mixture(rt, w, hid, F, E, top, FS, vocab)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(n, hid, generator=g).to(dtype)
    ids = torch.randint(0, vocab, (n,), generator=g)

    class Ctx:
        token_ids = i32(ids.tolist())
    got = part.forward(x.to(DEV), Ctx).clone()
    want = plain.table_mixture(x.double(), ids, {k: (v.double() if v.is_floating_point() else v) for k, v in w.items()}, "m.", f)
    close(got, want, 3e-5 if dtype == torch.float32 else 2e-2, "mixture")
    order = torch.randperm(n, generator=g)
    Ctx.token_ids = i32(ids[order].tolist())
    again = part.forward(x[order].to(DEV).contiguous(), Ctx)
    assert torch.equal(again.cpu(), got.cpu()[order])
    # the table's choice as lists and as a dense matrix
    ops = rt.ops
    dense = torch.empty(n, E, device=DEV)
    chosen, weights = torch.empty(n, top, dtype=torch.int32, device=DEV), torch.empty(n, top, device=DEV)
    ops.moe_table_route(Ctx.token_ids, w["m.table"].to(DEV), E, dense, chosen, weights)
    assert torch.equal(chosen.cpu(), w["m.table"][ids[order]]) and float((weights - 1.0 / top).abs().max()) < 1e-7
    assert torch.allclose(dense.sum(1).cpu(), torch.ones(n)) and int((dense > 0).sum()) == n * top


@pytest.mark.parametrize("n", [1, 7, 70, 300])
@pytest.mark.parametrize("hid, F, E, top, FS", [(64, 32, 5, 2, 96), (96, 64, 12, 1, 0), (32, 160, 3, 3, 32)])
def test_chosen_pairs_only_against_all_experts(n, hid, F, E, top, FS):
    """bfloat16 with sizes the MFMA kernels serve: the products over the chosen pairs only (the shared expert then runs as
    two products of its own and is added) give what computing every expert gives, and what the plain mixture gives."""
    dtype, vocab = torch.bfloat16, 90
    w, f = mixture_case(hid, F, E, top, FS, vocab, seed=n + E)
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, hid, generator=g).to(dtype)
    ids = torch.randint(0, vocab, (n,), generator=g)

    class Ctx:
        token_ids = i32(ids.tolist())
    outs = {}
    for grouped in (True, False):
        rt = runtime(dtype)
        part = build_mixture(rt, w, hid, F, E, top, FS, vocab, grouped=grouped, grouped_max_rows=1e9, grouped_min_weight=0)
        assert part.shared_packed == (bool(FS) and not grouped)
        rt.ops.ledger = []
        outs[grouped] = part.forward(x.to(DEV), Ctx).clone()
        torch.cuda.synchronize()
        assert ("mv_moe_grouped" in [e[0] for e in rt.ops.ledger]) == grouped
        rt.ops.ledger = None
    want = plain.table_mixture(x.double(), ids, {k: (v.double() if v.is_floating_point() else v) for k, v in w.items()}, "m.", f)
    close(outs[True], want, 2e-2, "chosen pairs only against the plain mixture")
    close(outs[True], outs[False].double(), 2e-2, "chosen pairs only against all experts")


@pytest.mark.parametrize("M", [1, 3, 8])
@pytest.mark.parametrize("N, K", [(1024, 16384), (512, 20480), (1024, 25344)])
def test_products_against_weights_with_long_rows(M, N, K):
    """The down matrices of a mixture's experts side by side are a weight with very long rows; steps of few rows send it
    to the tiled product, whose workgroups split the row."""
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(M + N)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(torch.bfloat16).to(DEV)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.ledger = []
    done = ops.gemm(a, w, out)
    if done is not None and not isinstance(done, torch.Tensor):
        done.materialize()
    torch.cuda.synchronize()
    assert [e[0] for e in ops.ledger][:1] == ["mv_gemm_tile"], [e[0] for e in ops.ledger]
    ops.ledger = None
    close(out, a.double() @ w.double().T, 1e-2, "long rows")
