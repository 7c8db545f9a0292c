"""The kernels of the recurrent mixers, of the general preparation of queries, keys and values, of capped attention
scores, of the norm behind and in front of a sublayer, of grouped sigmoid routing and of the clamped experts against
their plain torch twins, in float32 and in bfloat16, on sizes that are no multiples of anything."""
import numpy as np
import pytest
import torch

from llmserver_amd.parts.attention import build_attention_plan
from test_latent_experts_kernels_gpu import batch, close
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from llmserver_amd.kernels import default_ops
    return default_ops()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [8, 100, 1027, 4400])
def test_norm_add_norm_with_and_without_a_second_result_and_a_following_norm(ops, dtype, width):
    print(f"norm_add_norm {dtype} {width}", flush=True)
    twin = TorchOps()
    n = 7
    x = torch.randn(n, width, device="cuda")
    y, y2 = (3 * torch.randn(n, width, device="cuda")).to(dtype), torch.randn(n, width, device="cuda").to(dtype)
    w, w2 = 1 + 0.2 * torch.randn(width, device="cuda"), 1 + 0.2 * torch.randn(width, device="cuda")
    for second in (False, True):
        for following in (False, True):
            outs = [torch.empty(n, width, device="cuda") for _ in range(2)]
            normed = [torch.zeros(n, width, device="cuda", dtype=dtype) for _ in range(2)]
            for which, (o, nm) in zip((ops, twin), zip(outs, normed)):
                which.norm_add_norm(x, y, w, 1e-5, o, w2 if following else None, 3e-6, nm if following else None,
                                    y2 if second else None, (0.8, -1.3) if second else None)
            close(outs[0], outs[1], torch.float32, "sum")
            close(normed[0], normed[1], dtype, "following norm")
    table = torch.randn(19, width, device="cuda").to(dtype)
    ids = torch.randint(0, 19, (n,), device="cuda", dtype=torch.int32)
    wide = torch.empty(n, width, device="cuda")
    ops.embedding_wide(table, ids, wide)
    assert torch.equal(wide, table[ids.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_shift_over_steps_of_unequal_portions(ops, dtype):
    """Three requests go through steps of unequal portions; kernel and twin keep their own states, which must agree."""
    print(f"token_shift {dtype}", flush=True)
    twin = TorchOps()
    width, offset, mixes = 70, 5, 3
    mu = torch.randn(mixes, width, device="cuda")
    states = [torch.randn(5, offset + width + 2, device="cuda") for _ in range(2)]          # (a slot's leftovers must not be read)
    states[1].copy_(states[0])
    slots = torch.tensor([3, 0, 2], dtype=torch.int32, device="cuda")
    firsts = [0, 0, 0]
    for lengths in ([4, 1, 2], [1, 1, 1], [3, 0, 5], [1, 1, 1], [2, 7, 1]):
        rows = [r for r, n in enumerate(lengths) if n]
        token_row, positions, row_start, row_len, _ = batch([lengths[r] for r in rows], [firsts[r] for r in rows], "cuda")
        n = sum(lengths)
        h = torch.randn(n, width, device="cuda").to(dtype)
        outs = [torch.empty(mixes, n, width, device="cuda", dtype=dtype) for _ in range(2)]
        single = all(lengths[r] == 1 for r in rows)
        for which, state, out in zip((ops, twin), states, outs):
            which.token_shift(h, mu, state, offset, slots[rows].contiguous(), token_row, positions, row_start, out, keep=single)
            if not single:
                which.token_shift_keep(h, state, offset, slots[rows].contiguous(), row_start, row_len)
        close(outs[0], outs[1], dtype, f"mixes {lengths}")
        assert torch.equal(states[0], states[1])
        firsts = [f + n for f, n in zip(firsts, lengths)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,mode", [(3, 24, 40, "sigmoid_root"), (2, 64, 64, "double_exp"), (5, 7, 100, "sigmoid_root"),
                                                 (1, 130, 9, "double_exp"), (2, 300, 65, "sigmoid_root")])
def test_linear_recurrence_over_steps_and_slots(ops, dtype, heads, dim, vdim, mode):
    """Rows of unequal portions, an empty row, single tokens; the state travels in slots of a tensor that holds other
    things before it; a request that starts again in a used slot starts from zeros."""
    print(f"linear_recurrence {dtype} {heads} {dim} {vdim} {mode}", flush=True)
    twin = TorchOps()
    offset = 11
    size = heads * dim * vdim
    states = [torch.randn(4, offset + size, device="cuda") for _ in range(2)]
    states[1].copy_(states[0])
    slots = torch.tensor([2, 0, 3], dtype=torch.int32, device="cuda")
    bonus = torch.randn(heads, dim, device="cuda") if mode == "double_exp" else None
    bias = torch.randn(heads * dim, device="cuda")
    firsts = [0, 0, 0]
    for step, lengths in enumerate(([5, 1, 37], [1, 1, 1], [18, 0, 2], [1, 1, 1], [2, 40, 1])):
        if step == 3:
            firsts[1] = 0                          # the second request ends; another one starts in its slot
        token_row, positions, row_start, row_len, row_ctx = batch(lengths, firsts, "cuda")
        n = sum(lengths)
        proj = (0.5 * torch.randn(n, 2 * heads * dim + heads * vdim + 3, device="cuda")).to(dtype)
        q, k, v = proj[:, :heads * dim], proj[:, heads * dim:2 * heads * dim], proj[:, 2 * heads * dim:2 * heads * dim + heads * vdim]
        decay = 2 * torch.randn(n, heads * dim, device="cuda")
        outs = [torch.zeros(n, heads * vdim, device="cuda") for _ in range(2)]
        for which, state, out in zip((ops, twin), states, outs):
            which.linear_recurrence(q, k, v, decay, bias, mode, 4.0, bonus, 0.3, state, offset, slots, row_start, row_len, row_ctx, out,
                                    heads, dim, vdim)
        close(outs[0], outs[1], torch.float32, f"read-out, step {step}")
        close(states[0], states[1], torch.float32, f"state, step {step}")
        assert torch.equal(states[0][:, :offset], states[1][:, :offset]) and torch.equal(states[0][1], states[1][1])
        firsts = [f + n for f, n in zip(firsts, lengths)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_recurrence_does_not_depend_on_how_its_tokens_are_cut(ops, dtype):
    """The same bits, state and read-out, whether 50 tokens come at once, in portions or one by one."""
    heads, dim, vdim, n = 2, 48, 32, 50
    proj = torch.randn(n, 2 * heads * dim + heads * vdim, device="cuda").to(dtype)
    q, k, v = proj[:, :heads * dim], proj[:, heads * dim:2 * heads * dim], proj[:, 2 * heads * dim:]
    decay = torch.randn(n, heads * dim, device="cuda")
    make = lambda a: torch.tensor(a, dtype=torch.int32, device="cuda")
    results = []
    for cuts in ([50], [7, 16, 1, 26], [1] * 50):
        state = torch.zeros(1, heads * dim * vdim, device="cuda")
        out = torch.zeros(n, heads * vdim, device="cuda")
        at = 0
        for count in cuts:
            piece = slice(at, at + count)
            ops.linear_recurrence(q[piece], k[piece], v[piece], decay[piece].contiguous(), None, "sigmoid_root", 16.0, None, 1.0, state, 0,
                                  make([0]), make([0]), make([count]), make([at + count]), out[piece], heads, dim, vdim)
            at += count
        results.append((out, state))
    for out, state in results[1:]:
        assert torch.equal(out, results[0][0]) and torch.equal(state, results[0][1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_norm_gate_tanh_and_scaled_sum(ops, dtype):
    twin = TorchOps()
    n, heads, vdim = 9, 5, 70
    x = 4 * torch.randn(n, heads * vdim, device="cuda")
    wide = torch.randn(n, heads * vdim + 6, device="cuda").to(dtype)
    gate = wide[:, 3:3 + heads * vdim]
    for per_channel in (False, True):
        weight = 1 + 0.3 * torch.randn(heads * vdim if per_channel else vdim, device="cuda")
        outs = [torch.empty(n, heads * vdim, device="cuda", dtype=dtype) for _ in range(2)]
        for which, out in zip((ops, twin), outs):
            which.heads_norm_gate(x, weight, per_channel, 1e-5, gate, out, heads, vdim)
        close(outs[0], outs[1], dtype, "heads_norm_gate")
    a, b = wide.clone(), wide.clone()
    ops.tanh_(a)
    twin.tanh_(b)
    close(a, b, dtype, "tanh")
    outs = [torch.empty_like(wide) for _ in range(2)]
    for which, out in zip((ops, twin), outs):
        which.scaled_sum(wide, 0.8, a, 0.9, out)
    close(outs[0], outs[1], dtype, "scaled_sum")


def staged_plan(plan, device):
    staged = {"items": plan.items, "item_slot": plan.item_slot, "merges": plan.merges, "tiles": plan.tiles}
    out = {name: torch.tensor(value, dtype=torch.int32, device=device) for name, value in staged.items()}
    out.update(n_items=len(plan.items), n_merges=len(plan.merges), n_slots=plan.n_slots, n_tiles=len(plan.tiles),
               tiles_per_workgroup=plan.tiles_per_workgroup, tile_halves=int(plan.tile_halves), merge_in_workgroup=0,
               most_splits=int(plan.merges[:, 3].max()) if len(plan.merges) else 0)
    if plan.tile_slots is not None:
        out["tile_slots"] = torch.tensor(plan.tile_slots, dtype=torch.int32, device=device)
    return out


class _Ctx:
    @staticmethod
    def empty(shape, dtype=None):
        return torch.empty(shape, device="cuda", dtype=dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_q,n_kv,dim,vdim,pairs,window,cap", [(6, 2, 24, 40, 5, 9, 3.0), (8, 1, 64, 64, 16, 72, 50.0), (3, 3, 10, 7, 0, None, 0.7),
                                                                (4, 2, 48, 48, 24, 33, 2.0)])
def test_prepared_queries_keys_values_and_capped_windowed_attention_with_sinks(ops, dtype, n_q, n_kv, dim, vdim, pairs, window, cap):
    """Portions behind cached keys, a long prompt (workgroup tiles) and single tokens, through scrambled pages."""
    print(f"qkv_prepare + attention {dtype} {n_q} {n_kv} {dim} {vdim} {pairs} {window} {cap}", flush=True)
    twin = TorchOps()
    page, row = 8, -(-max(dim, vdim) // 16) * 16
    lengths, firsts = [150, 1, 1, 20], [0, 77, 9, 60]
    pages_needed = [-(-(f + n) // page) for f, n in zip(firsts, lengths)]
    order = torch.randperm(sum(pages_needed) + 3).tolist()
    table = np.full((4, max(pages_needed)), -1, dtype=np.int32)
    for r, count in enumerate(pages_needed):
        table[r, :count] = [order.pop() for _ in range(count)]
    table = torch.tensor(table, device="cuda")
    caches = [[(torch.randn(sum(pages_needed) + 3, n_kv, *shape, device="cuda") * 0.5).to(dtype) for shape in ((page, row), (row, page))] for _ in range(2)]
    caches[1][0].copy_(caches[0][0])
    caches[1][1].copy_(caches[0][1])
    # what stands before the portions: keys and values of earlier steps, written by the same kernel
    weights = (1 + 0.2 * torch.randn(dim, device="cuda"), 1 + 0.2 * torch.randn(dim, device="cuda"))
    sinks = torch.randn(n_q, device="cuda")
    inv_freq = torch.tensor([100.0 ** (-2.0 * i / max(2 * pairs, 2)) for i in range(pairs)], device="cuda")
    columns = (n_q + n_kv) * dim + n_kv * vdim
    for phase, (lens, starts) in enumerate((([f for f in firsts], [0] * 4), (lengths, firsts))):
        rows = [r for r, n in enumerate(lens) if n]
        token_row, positions, row_start, row_len, row_ctx = batch([lens[r] for r in rows], [starts[r] for r in rows], "cuda")
        n = sum(lens)
        qkv = torch.randn(n, columns, device="cuda").to(dtype)
        cos_sin = twin.rotary_table(positions, inv_freq) if pairs else None
        sub_table = table[rows].contiguous()
        qs = [torch.empty(n, n_q * row, device="cuda", dtype=dtype) for _ in range(2)]
        for which, (keys, values), q in zip((ops, twin), caches, qs):
            which.qkv_prepare(qkv, keys, values, sub_table, token_row, positions, weights[0], weights[1], 1e-5, cos_sin, page, n_q, n_kv,
                              dim, vdim, q, True)
        close(qs[0], qs[1], dtype, "queries")
        close(caches[0][0], caches[1][0], dtype, "key pages")
        close(caches[0][1], caches[1][1], dtype, "value pages")
        if phase == 0:
            continue
        plan = build_attention_plan(row_len.cpu().numpy(), row_ctx.cpu().numpy(), n_q // n_kv, n_kv, window,
                                    workgroup_tiles=ops.attention_workgroup_tiles(dtype, row, page),
                                    tuning=ops.attention_tuning_for(dtype, row))
        outs = [torch.zeros(n, n_q * row, device="cuda", dtype=dtype) for _ in range(2)]
        ops.paged_attention(qs[1], outs[0], caches[1][0], caches[1][1], sub_table, row_start, row_len, row_ctx, staged_plan(plan, "cuda"),
                            dim ** -0.5, window, page, n_q, n_kv, row, _Ctx, sinks=sinks, softcap=cap)
        twin.paged_attention(qs[1], outs[1], caches[1][0], caches[1][1], sub_table, row_start, row_len, row_ctx, None, dim ** -0.5, window,
                             page, n_q, n_kv, row, None, sinks=sinks, softcap=cap)
        close(outs[0], outs[1], dtype, "attention")
        assert float(outs[0].view(n, n_q, row)[:, :, vdim:].abs().max()) == 0.0 if row > vdim else True


@pytest.mark.parametrize("experts,top,groups", [(16, 2, (2, 1)), (12, 3, (4, 2)), (9, 4, None), (64, 6, (8, 3)), (6, 1, (6, 1)), (5, 5, (1, 1))])
def test_sigmoid_routing_with_groups(ops, experts, top, groups):
    twin = TorchOps()
    for n in (3, 40):
        x = torch.randn(n, 50, device="cuda")
        router = torch.randn(experts, 50, device="cuda")
        chosen = [torch.zeros(n, top, dtype=torch.int32, device="cuda") for _ in range(2)]
        weights = [torch.zeros(n, top, device="cuda") for _ in range(2)]
        for which, c, w in zip((ops, twin), chosen, weights):
            which.route_experts(x, router, top, c, w, scoring="sigmoid", groups=groups)
        assert torch.equal(chosen[0], chosen[1])
        close(weights[0], weights[1], torch.float32, "scores")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [3, 70])
def test_clamped_experts_per_pair_and_sorted(ops, dtype, n):
    twin = TorchOps()
    width, inter, experts, top, limit = 64, 96, 8, 2, 0.6
    x = torch.randn(n, width, device="cuda").to(dtype)
    gate_up = (0.3 * torch.randn(experts, 2 * inter, width, device="cuda")).to(dtype)
    down = (0.3 * torch.randn(experts, width, inter, device="cuda")).to(dtype)
    chosen = torch.stack([torch.randperm(experts)[:top] for _ in range(n)]).to(device="cuda", dtype=torch.int32)
    weights = torch.rand(n, top, device="cuda")
    hidden = [torch.empty(n * top, inter, device="cuda", dtype=dtype) for _ in range(2)]
    for which, h in zip((ops, twin), hidden):
        which.experts_gate_up(x, gate_up, chosen, h, activation="clamped", limit=limit)
    close(hidden[0], hidden[1], dtype, "clamped activation")
    want = torch.empty(n, width, device="cuda")
    twin.experts_down(hidden[1], down, chosen, weights, want)
    got = torch.empty(n, width, device="cuda")
    if ops.experts_sorted(x, gate_up, down, chosen, weights, got, activation="clamped", limit=limit):
        close(got, want, dtype, "sorted experts")
    else:
        assert dtype == torch.float32 or n * top <= experts


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_activation_with_the_tanh_form_of_gelu(ops, dtype):
    twin = TorchOps()
    gate_up = (2 * torch.randn(13, 2 * 90, device="cuda")).to(dtype)
    outs = [torch.empty(13, 90, device="cuda", dtype=dtype) for _ in range(2)]
    for which, out in zip((ops, twin), outs):
        which.swiglu(gate_up, out, activation="gelu_tanh")
    close(outs[0], outs[1], dtype, "gelu_tanh")


def test_a_recurrence_with_heads_of_128_channels_is_recorded_into_a_graph_and_replayed(ops):
    """Heads of 128 key channels take more LDS than a kernel gets by default; the launch must be nothing but a launch,
    so that a captured step can hold it.  Every replay (inputs changed in place between them, eager work and
    synchronisations in between) equals the eager result."""
    heads, dim, vdim, n = 2, 128, 128, 40
    make = lambda a: torch.tensor(a, dtype=torch.int32, device="cuda")
    proj = torch.randn(n, 3 * heads * dim, device="cuda").to(torch.bfloat16)
    q, k, v = proj[:, :heads * dim], proj[:, heads * dim:2 * heads * dim], proj[:, 2 * heads * dim:]
    decay = torch.randn(n, heads * dim, device="cuda")
    bonus = torch.randn(heads, dim, device="cuda")
    state = torch.zeros(2, heads * dim * vdim, device="cuda")
    out = torch.zeros(n, heads * vdim, device="cuda")
    args = (q, k, v, decay, None, "double_exp", 1.0, bonus, 1.0, state, 0, make([1]), make([0]), make([n]), make([n]), out, heads, dim, vdim)
    ops.linear_recurrence(*args)                      # (eager first, as every captured step runs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.linear_recurrence(*args)
    twin = TorchOps()
    for replay in range(3):
        proj.copy_(torch.randn(n, 3 * heads * dim, device="cuda").to(torch.bfloat16))
        decay.copy_(torch.randn(n, heads * dim, device="cuda"))
        graph.replay()
        torch.cuda.synchronize()
        want, want_state = torch.zeros_like(out), torch.zeros_like(state)
        twin.linear_recurrence(q, k, v, decay, None, "double_exp", 1.0, bonus, 1.0, want_state, 0, make([1]), make([0]), make([n]), make([n]),
                               want, heads, dim, vdim)
        close(out, want, torch.float32, f"replay {replay}")
        close(state, want_state, torch.float32, f"state after replay {replay}")
