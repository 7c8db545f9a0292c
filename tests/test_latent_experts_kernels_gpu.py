"""The kernels of the 32-bit residual stream, of attention over a latent and of routed experts against their plain
torch twins, in float32 and in bfloat16, on sizes that are no multiples of anything."""
import numpy as np
import pytest
import torch

from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from llmserver_amd.kernels import default_ops
    return default_ops()


def close(got, want, dtype, what):
    got, want = got.float().cpu(), want.float().cpu()
    tolerance = 2e-5 if dtype == torch.float32 else 1.2e-2
    size = max(1.0, float(want.abs().max()))
    assert float((got - want).abs().max()) <= tolerance * size, (what, float((got - want).abs().max()), size)


def batch(lengths, firsts, device):
    """Rows of ``lengths`` tokens whose first tokens stand at positions ``firsts``."""
    token_row = np.concatenate([np.full(n, r) for r, n in enumerate(lengths)])
    positions = np.concatenate([np.arange(f, f + n) for f, n in zip(firsts, lengths)])
    row_start = np.concatenate([[0], np.cumsum(lengths)[:-1]])
    row_ctx = np.asarray(firsts) + np.asarray(lengths)
    make = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=device)
    return make(token_row), make(positions), make(row_start), make(lengths), make(row_ctx)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [8, 100, 257, 1024])
def test_embedding_norm_and_norm_rows(ops, dtype, width):
    print(f"embedding_norm {dtype} {width}", flush=True)
    twin = TorchOps()
    table = torch.randn(37, width, device="cuda").to(dtype)
    ids = torch.randint(0, 37, (11,), device="cuda", dtype=torch.int32)
    weight = 1 + 0.1 * torch.randn(width, device="cuda")
    got, want = torch.empty(11, width, device="cuda"), torch.empty(11, width, device="cuda")
    ops.embedding_norm(table, ids, weight, 1e-5, got)
    twin.embedding_norm(table, ids, weight, 1e-5, want)
    close(got, want, torch.float32, "embedding_norm")
    rows = torch.tensor([7, 0, 3], dtype=torch.int32, device="cuda")
    for picked, n in ((rows, 3), (None, 11)):
        out_got, out_want = torch.empty(n, width, device="cuda", dtype=dtype), torch.empty(n, width, device="cuda", dtype=dtype)
        ops.norm_rows(got, picked, weight, 1e-5, out_got)
        twin.norm_rows(want, picked, weight, 1e-5, out_want)
        close(out_got, out_want, dtype, "norm_rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_short_convolution_with_state_over_steps(ops, dtype, taps):
    """Three requests go through several steps of unequal portions (shorter than the taps reach, too); the state that
    one step leaves is what the next one reads.  Kernel and twin start from the same zeros and must stay together."""
    print(f"short_conv {dtype} taps {taps}", flush=True)
    twin, width, slots = TorchOps(), 70, 5
    weight = torch.randn(width, taps, device="cuda")
    states = [torch.zeros(slots, taps - 1, width, device="cuda") if taps > 1 else None for _ in range(2)]
    slot_of = torch.tensor([3, 0, 4], dtype=torch.int32, device="cuda")
    firsts = [0, 0, 0]
    for lengths in ([1, 4, 9], [1, 1, 1], [2, 1, 7], [1, 3, 1], [6, 1, 2]):
        token_row, positions, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
        x = torch.randn(sum(lengths), width, device="cuda")
        outs = [torch.empty(sum(lengths), width, device="cuda", dtype=dtype) for _ in range(2)]
        for which, state, out in ((ops, states[0], outs[0]), (twin, states[1], outs[1])):
            single = max(lengths) == 1 and state is not None       # one token a row: the kernel may move the state on itself
            which.short_conv(x, weight, state, slot_of, token_row, positions, row_start, out, keep=single)
            if state is not None and not single:
                which.short_conv_keep(x, state, slot_of, row_start, row_len, row_ctx)
        close(outs[0], outs[1], dtype, f"short_conv {lengths}")
        if taps > 1:
            close(states[0], states[1], torch.float32, f"state after {lengths}")
        firsts = [f + n for f, n in zip(firsts, lengths)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("y_float32", [False, True])
def test_scaled_norm_add_with_and_without_history(ops, dtype, y_float32):
    print(f"scaled_norm_add {dtype} {y_float32}", flush=True)
    twin, n, width = TorchOps(), 9, 130
    x = torch.randn(n, width, device="cuda")
    y = torch.randn(n, width, device="cuda").to(torch.float32 if y_float32 else dtype)
    weight, scale = 1 + 0.1 * torch.randn(width, device="cuda"), torch.randn(width, device="cuda")
    for history_states, before in ((None, 0), (4, 1), (4, 3)):
        results = []
        for which in (ops, twin):
            out, rounded = torch.empty(n, width, device="cuda"), torch.empty(n, width, device="cuda", dtype=dtype)
            extra = {}
            if history_states:
                generator = torch.Generator(device="cuda").manual_seed(5)
                extra = {"history": torch.randn(history_states, n, width, device="cuda", generator=generator), "before": before,
                         "mix": torch.tensor([0.5, -1.25, 2.0, 0.75], device="cuda")[:before + 1].contiguous()}
            which.scaled_norm_add(x, y, weight, scale if before != 1 else None, 1e-5, out, rounded=rounded, **extra)
            results.append((out, rounded, extra.get("history")))
        close(results[0][0], results[1][0], torch.float32, "out")
        close(results[0][1], results[1][1], dtype, "rounded")
        if history_states:
            close(results[0][2], results[1][2], torch.float32, "history")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, rot_dim, rank, pairs", [(3, 8, 4, 20, 2), (5, 24, 16, 40, 8), (2, 16, 8, 56, 3)])
def test_latent_prepare_and_gate_heads(ops, dtype, heads, dim, rot_dim, rank, pairs):
    print(f"latent_prepare {dtype} {heads} {dim} {rot_dim} {rank} {pairs}", flush=True)
    twin, page_size = TorchOps(), 8
    row_width = -(-(rank + rot_dim) // 16) * 16
    lengths, firsts = [5, 1, 11], [3, 40, 0]
    token_row, positions, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
    n = sum(lengths)
    proj = torch.randn(n, heads * (dim + rot_dim) + rank + rot_dim + heads, device="cuda").to(dtype)
    q_latent = torch.randn(heads, n, rank, device="cuda").to(dtype)
    norm_weight = 1 + 0.1 * torch.randn(rank, device="cuda")
    angles = torch.randn(n, pairs, device="cuda") * 3
    cos_sin = torch.cat([torch.cos(angles), torch.sin(angles)], dim=1).contiguous()
    table = torch.tensor([[9, 2, -1, -1, -1, -1], [0, 1, 3, 4, 5, 6], [7, 8, -1, -1, -1, -1]], dtype=torch.int32, device="cuda")
    results = []
    for which in (ops, twin):
        keys = torch.full((10, 1, page_size, row_width), 7.0, device="cuda").to(dtype)
        values = torch.full((10, 1, row_width, page_size), 7.0, device="cuda").to(dtype)
        out_q = torch.empty(n, heads * row_width, device="cuda", dtype=dtype)
        which.latent_prepare(proj, q_latent, norm_weight, 1e-5, cos_sin, keys, values, table, token_row, positions, page_size, out_q,
                             heads, dim, rot_dim, rank, True)
        y = torch.randn(heads, n, 12, device="cuda", generator=torch.Generator(device="cuda").manual_seed(3)).to(dtype)
        gated, plain = torch.empty(n, heads * 12, device="cuda", dtype=dtype), torch.empty(n, heads * 12, device="cuda", dtype=dtype)
        which.gate_heads(y, proj, heads * (dim + rot_dim) + rank + rot_dim, gated)
        which.gate_heads(y, proj, -1, plain)
        # the same with the per-head products made inside the kernels (steps of few tokens go this way)
        generator = torch.Generator(device="cuda").manual_seed(4)
        up_keys = (torch.randn(heads, dim, rank, device="cuda", generator=generator) / dim ** 0.5).to(dtype)
        up_values = (torch.randn(heads, rank, 12, device="cuda", generator=generator) / rank ** 0.5).to(dtype)
        inside_q = torch.empty(n, heads * row_width, device="cuda", dtype=dtype)
        which.latent_prepare(proj, None, norm_weight, 1e-5, cos_sin, keys, values, table, token_row, positions, page_size, inside_q,
                             heads, dim, rot_dim, rank, False, up_keys=up_keys)
        inside_gated = torch.empty(n, heads * 12, device="cuda", dtype=dtype)
        which.gate_heads(None, proj, heads * (dim + rot_dim) + rank + rot_dim, inside_gated, mixed=out_q, up_values=up_values)
        results.append((keys, values, out_q, gated, plain, inside_q, inside_gated))
    for got, want, what in zip(results[0], results[1], ("keys", "values", "q", "gated", "ungated", "q made inside", "gated made inside")):
        close(got, want, dtype, what)
    assert torch.equal(results[0][0].transpose(2, 3)[results[0][0].transpose(2, 3) != 7], results[0][1][results[0][1] != 7])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts, top, width, inter", [(5, 1, 24, 10), (12, 2, 100, 36), (70, 6, 320, 64), (4, 4, 30, 7)])
def test_routed_experts(ops, dtype, experts, top, width, inter):
    print(f"experts {dtype} {experts} {top} {width} {inter}", flush=True)
    twin, n = TorchOps(), 13
    x = torch.randn(n, width, device="cuda").to(dtype)
    router = torch.randn(experts, width, device="cuda")
    router[1] = router[0]                                          # equal logits: the lower index wins
    gate_up = (torch.randn(experts, 2 * inter, width, device="cuda") / width ** 0.5).to(dtype)
    down = (torch.randn(experts, width, inter, device="cuda") / inter ** 0.5).to(dtype)
    results = []
    for which in (ops, twin):
        chosen = torch.empty(n, top, dtype=torch.int32, device="cuda")
        weights = torch.empty(n, top, device="cuda")
        which.route_experts(x, router, top, chosen, weights)
        hidden = torch.empty(n * top, inter, device="cuda", dtype=dtype)
        which.experts_gate_up(x, gate_up, chosen, hidden)
        out = torch.empty(n, width, device="cuda")
        which.experts_down(hidden, down, chosen, weights, out)
        results.append((chosen, weights, hidden, out))
    logits = x.float() @ router.t()
    for token in range(n):                                          # the same set, unless two logits are a rounding apart
        mine, theirs = set(results[0][0][token].tolist()), set(results[1][0][token].tolist())
        if mine != theirs:
            edge = torch.sort(logits[token], descending=True).values
            assert top < experts and float(edge[top - 1] - edge[top]) < 1e-4, (token, mine, theirs)
            return
    # (equal logits may come in either order; the kernel's order is the lower index first)
    tie = results[0][0][(results[0][0] <= 1).all(dim=1)] if top == 2 else None
    assert tie is None or all(row.tolist() == [0, 1] for row in tie)
    close(results[0][1].sort(dim=1).values, results[1][1].sort(dim=1).values, torch.float32, "weights")
    order = [results[i][0].long().argsort(dim=1) for i in range(2)]
    rows = [results[i][2].view(n, top, inter).gather(1, order[i][..., None].expand(-1, -1, inter)) for i in range(2)]
    close(rows[0], rows[1], dtype, "hidden")
    close(results[0][3], results[1][3], dtype, "out")


@pytest.mark.parametrize("experts, top, width, inter, tokens", [(5, 2, 64, 32, 40), (12, 3, 96, 160, 333), (70, 6, 192, 96, 200), (70, 6, 192, 96, 100), (40, 2, 64, 128, 90), (3, 1, 32, 64, 700)])
def test_sorted_expert_products_equal_the_per_pair_ones(ops, experts, top, width, inter, tokens):
    """Many tokens: the pairs sorted by expert and multiplied tile by tile give what every pair alone gives."""
    print(f"sorted experts {experts} {top} {width} {inter} {tokens}", flush=True)
    twin, dtype = TorchOps(), torch.bfloat16
    x = torch.randn(tokens, width, device="cuda").to(dtype)
    router = torch.randn(experts, width, device="cuda")
    if experts > 4:
        router[3] *= 0.0
        router[3] -= 100.0 * x.float().mean(dim=0)                 # an expert that (almost) nobody chooses
    gate_up = (torch.randn(experts, 2 * inter, width, device="cuda") / width ** 0.5).to(dtype)
    down = (torch.randn(experts, width, inter, device="cuda") / inter ** 0.5).to(dtype)
    chosen = torch.empty(tokens, top, dtype=torch.int32, device="cuda")
    weights = torch.empty(tokens, top, device="cuda")
    ops.route_experts(x, router, top, chosen, weights)
    out = torch.empty(tokens, width, device="cuda")
    assert ops.experts_sorted(x, gate_up, down, chosen, weights, out)
    hidden = torch.empty(tokens * top, inter, device="cuda", dtype=dtype)
    single = torch.empty(tokens, width, device="cuda")
    ops.experts_gate_up(x, gate_up, chosen, hidden)
    ops.experts_down(hidden, down, chosen, weights, single)
    close(out, single, dtype, "sorted against per pair")
    some = min(50, tokens)
    part = slice(0, some)
    want_hidden = torch.empty(some * top, inter, device="cuda", dtype=dtype)
    want = torch.empty(some, width, device="cuda")
    twin.experts_gate_up(x[part], gate_up, chosen[part], want_hidden)
    twin.experts_down(want_hidden, down, chosen[part], weights[part], want)
    close(out[part], want, dtype, "sorted against the twin")
    assert not ops.experts_sorted(x[:1], gate_up, down, chosen[:1], weights[:1], out[:1]) or top > experts


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_counts_once_however_the_keys_are_cut(ops, dtype):
    """Attention with a sink over one key-value head against the twin: a prompt whole (workgroups of tiles), single
    tokens behind long contexts (key ranges merged by a second launch and inside a workgroup), with a sink that
    outweighs every key, one that weighs nothing, and ordinary ones."""
    from llmserver_amd.engine.batch import Staging, StepContext
    from llmserver_amd.parts.attention import stage_attention_plan
    print(f"sinks {dtype}", flush=True)
    twin, heads, d, page_size = TorchOps(), 5, 48, 16
    sinks = torch.tensor([30.0, -30.0, 0.0, 1.5, -2.0], device="cuda")
    for lengths, firsts, static in (([300], [0], None), ([1, 1, 1], [700, 64, 1500], None), ([1, 1], [900, 300], 2048),
                                    ([1, 1, 1, 1], [100, 300, 17, 0], 512), ([40, 1, 3], [260, 33, 0], None)):
        token_row, positions, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
        n, rows = sum(lengths), len(lengths)
        pages_per_row = [-(-(f + c) // page_size) for f, c in zip(firsts, lengths)]
        width = max(pages_per_row) if static is None else static // page_size
        order = torch.randperm(sum(pages_per_row)).tolist()
        table = torch.full((rows, width), -1, dtype=torch.int32)
        for row, count in enumerate(pages_per_row):
            table[row, :count] = torch.tensor([order.pop() for _ in range(count)], dtype=torch.int32)
        table = table.cuda()
        keys = torch.randn(sum(pages_per_row), 1, page_size, d, device="cuda").to(dtype)
        values = keys.transpose(2, 3).contiguous()
        q = torch.randn(n, heads * d, device="cuda").to(dtype)
        ctx = StepContext(ops, "cuda", dtype, Staging("cuda"))
        ctx.page_size = page_size
        ctx.fill(np.zeros(n), positions.cpu().numpy(), token_row.cpu().numpy(), row_start.cpu().numpy(), row_len.cpu().numpy(),
                 row_ctx.cpu().numpy(), [], [table.cpu().numpy()], None, list(range(rows)))
        ctx.static_max_keys = static
        stage_attention_plan(ctx, "plan", heads, 1, d, None, lambda r, longest: "short" if longest <= 512 else None)
        ctx.upload()
        got, want = torch.empty(n, heads * d, device="cuda", dtype=dtype), torch.empty(n, heads * d, device="cuda", dtype=dtype)
        ops.paged_attention(q, got, keys, values, ctx.block_table(0), ctx.row_start, ctx.row_len, ctx.row_ctx, ctx.get_plan("plan"),
                            0.2, None, page_size, heads, 1, d, ctx, sinks=sinks)
        twin.paged_attention(q, want, keys, values, table, row_start, row_len, row_ctx, None, 0.2, None, page_size, heads, 1, d, None,
                             sinks=sinks)
        close(got, want, dtype, f"attention with sinks {lengths} {firsts}")
        assert float(got.view(n, heads, d)[:, 0].abs().max()) < 1e-3          # the first head's sink takes nearly all the weight
