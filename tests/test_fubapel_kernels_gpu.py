"""The kernels behind the Fubapel mixers, each alone against its plain reference (``kernel_refs``) on the same inputs,
in float32 and bfloat16, at sizes that are no multiples of anything; and inputs made so that one fault shows: a single
key that must win (far back, on both sides of a page border, the newest, and one that is not yet visible), a sink that
takes all or nothing of the weight, a state that must survive steps and slots."""
import pytest
import torch

import kernel_refs as refs
from qil_amd import ops

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def to(device, *tensors):
    return [None if t is None else t.to(device) for t in tensors]


def close(actual, expected, dtype, scale=1.0):
    tolerance = dict(atol=2e-5 * scale, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2 * scale, rtol=2e-2)
    torch.testing.assert_close(actual.float().cpu(), expected.float(), **tolerance)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('centre', [True, False])
@pytest.mark.parametrize('width', [40, 257, 1100])
def test_norm_with_scaled_add(dtype, centre, width):
    g = torch.Generator().manual_seed(width)
    n = 7
    stream = torch.randn(n, width, generator=g) * 3 + 1.5
    weight = 1 + 0.1 * torch.randn(width, generator=g)
    delta = torch.randn(n, width, generator=g).to(dtype)
    parts = ops.Partials(torch.randn(3, n, width, generator=g).cuda())
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
    for d_gpu, d_cpu in ((delta.cuda(), delta), (parts, parts.tensor.cpu().sum(0)), (None, None)):
        s_gpu, s_cpu = stream.clone().cuda(), stream.clone()
        got = ops.add_norm(s_gpu, d_gpu, weight.cuda(), 1e-5, dtype, centre=centre, delta_scale=0.7)
        want = refs.add_norm(s_cpu, d_cpu, weight, 1e-5, dtype, centre=centre, delta_scale=0.7)
        close(got, want, dtype)
        close(s_gpu, s_cpu, torch.float32)                                     # the stream holds the sum
        before = s_gpu.clone()
        got = ops.rows_norm(s_gpu, d_gpu, rows.cuda(), weight.cuda(), 1e-5, dtype, centre=centre, delta_scale=1.3)
        close(got, refs.rows_norm(s_cpu, d_cpu, rows, weight, 1e-5, dtype, centre=centre, delta_scale=1.3), dtype)
        assert torch.equal(before, s_gpu)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('interleaved', [False, True])
def test_clamped_gate(dtype, interleaved):
    g = torch.Generator().manual_seed(1)
    n, inner = 5, 48
    both = (torch.randn(n, 2 * inner, generator=g) * 3).to(dtype)               # values on both sides of the limits
    for activation, limit, alpha in (('clamped_swish', 1.25, 1.702), ('silu', 0.0, 1.0)):
        got = ops.gated_act(both.cuda(), dtype, activation=activation, limit=limit, alpha=alpha, interleaved=interleaved)
        close(got, refs.gated_act(both, dtype, activation=activation, limit=limit, alpha=alpha, interleaved=interleaved), dtype, 4.0)
    parts = torch.randn(2, n, 2 * inner, generator=g) * 2
    got = ops.gated_act(ops.Partials(parts.cuda()), dtype, activation='clamped_swish', limit=0.5, alpha=1.702, interleaved=interleaved)
    close(got, refs.gated_act(parts.sum(0), dtype, activation='clamped_swish', limit=0.5, alpha=1.702, interleaved=interleaved), dtype)


def test_the_feed_forward_part_uses_the_gate_it_is_given():
    from qil_amd.parts import GatedMLP
    g = torch.Generator().manual_seed(2)
    width, inner, n = 24, 40, 6
    part = GatedMLP(width=width, intermediate=inner, activation='clamped_swish', limit=0.8, alpha=1.702, dtype=torch.float32)
    gate, up, down = (torch.randn(s, generator=g) for s in ((inner, width), (inner, width), (width, inner)))
    for name, t in (('gate_proj.weight', gate), ('up_proj.weight', up), ('down_proj.weight', down)):
        part.set_param(name, t.cuda())
    part.finalize()
    h = torch.randn(n, width, generator=g)
    out = part.forward(h.cuda())
    out = out.sum() if isinstance(out, ops.Partials) else out
    a, b = (h @ gate.t()).clamp(max=0.8), (h @ up.t()).clamp(-0.8, 0.8)
    close(out, (a * torch.sigmoid(1.702 * a) * (b + 1)) @ down.t(), torch.float32, 4.0)


@pytest.mark.parametrize('dtype', DTYPES)
def test_latent_prepare_and_query(dtype):
    g = torch.Generator().manual_seed(3)
    n, q_rank, rank, rot, heads, dim, page = 9, 14, 20, 6, 5, 12, 4
    freq = torch.tensor([300.0 ** (-2 * i / rot) for i in range(rot // 2)], dtype=torch.float32)
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 1000, 7, 8], dtype=torch.int32)
    slots = torch.tensor([11, 3, 0, 30, 31, 8, 5, 6, 19], dtype=torch.int32)
    down = (torch.randn(n, q_rank + rank + rot, generator=g) * 2).to(dtype)
    wq, wc = 1 + 0.2 * torch.randn(q_rank, generator=g), 1 + 0.2 * torch.randn(rank, generator=g)
    lat_c, rope_c = torch.zeros(8, page, rank, dtype=dtype), torch.zeros(8, page, rot, dtype=dtype)
    lat_g, rope_g = lat_c.clone().cuda(), rope_c.clone().cuda()
    common = dict(q_rank=q_rank, rank=rank, rot=rot, eps=1e-5, dtype=dtype)
    want = refs.latent_prepare(down, q_weight=wq, c_weight=wc, frequencies=freq, positions=positions, slots=slots,
                               latent=lat_c, rope=rope_c, **common)
    got = ops.latent_prepare(down.cuda(), q_weight=wq.cuda(), c_weight=wc.cuda(), frequencies=freq.cuda(),
                             positions=positions.cuda(), slots=slots.cuda(), latent=lat_g, rope=rope_g, **common)
    close(got, want, dtype, 3.0), close(lat_g, lat_c, dtype, 3.0), close(rope_g, rope_c, dtype, 6.0)
    split = ops.Partials(torch.stack([down.float() * 0.25, down.float() * 0.75]).cuda())      # the same values as partial sums
    again = ops.latent_prepare(split, q_weight=wq.cuda(), c_weight=wc.cuda(), frequencies=freq.cuda(),
                               positions=positions.cuda(), slots=None, latent=lat_g, rope=rope_g, **common)
    close(again, want, dtype, 3.0)
    q = torch.randn(n, heads * (dim + rot), generator=g).to(dtype)
    k_up = torch.randn(heads, dim, rank, generator=g).to(dtype)
    want = refs.latent_query(q, k_up, heads=heads, dim=dim, rot=rot, rank=rank, frequencies=freq, positions=positions)
    got = ops.latent_query(q.cuda(), k_up.cuda(), heads=heads, dim=dim, rot=rot, rank=rank, frequencies=freq.cuda(),
                           positions=positions.cuda())
    close(got, want, torch.float32, 10.0)
    x = torch.randn(n, heads * rank, generator=g)
    v_up = torch.randn(heads, rank, 7, generator=g).to(dtype)
    close(ops.head_product(x.cuda(), v_up.cuda(), heads=heads, out_dtype=dtype),
          refs.head_product(x, v_up, heads=heads, out_dtype=dtype), dtype, 10.0)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('sizes', [dict(n=3, heads=3, k=40, o=64), dict(n=9, heads=2, k=130, o=72), dict(n=32, heads=1, k=7, o=16),
                                   dict(n=33, heads=2, k=40, o=64), dict(n=5, heads=4, k=33, o=20),
                                   dict(n=300, heads=3, k=40, o=64), dict(n=257, heads=2, k=33, o=20)])
def test_a_product_per_head_for_few_and_for_many_rows(dtype, sizes):
    """Few rows with outputs in whole groups of eight take the kernel that splits k, many rows in bfloat16 the batched
    product of the GPU BLAS, other shapes the plain kernel."""
    n, heads, k, o = sizes['n'], sizes['heads'], sizes['k'], sizes['o']
    g = torch.Generator().manual_seed(n * o)
    x = torch.randn(n, heads * k, generator=g)
    w = torch.randn(heads, k, o, generator=g).to(dtype)
    close(ops.head_product(x.cuda(), w.cuda(), heads=heads, out_dtype=dtype),
          refs.head_product(x, w, heads=heads, out_dtype=dtype), dtype, 10.0)


def paged(n_tokens, page, rank, rot, dtype, g, order):
    """Caches of one sequence of n_tokens whose pages lie in the given order among others filled with NaN."""
    pages = -(-n_tokens // page)
    latent = torch.full((len(order) + 3, page, rank), float('nan')).to(dtype)
    rope = torch.full((len(order) + 3, page, rot), float('nan')).to(dtype)
    table = torch.tensor(order[:pages], dtype=torch.int32)
    c, r = torch.randn(n_tokens, rank, generator=g).to(dtype), torch.randn(n_tokens, rot, generator=g).to(dtype)
    keys = torch.arange(n_tokens)
    slots = table.long()[keys // page] * page + keys % page
    latent.view(-1, rank)[slots], rope.view(-1, rot)[slots] = c, r
    return latent, rope, table, c, r


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('sizes', [dict(heads=5, rank=20, rot=6, page=4), dict(heads=1, rank=130, rot=2, page=16),
                                   dict(heads=40, rank=96, rot=32, page=8)])
def test_latent_attention_against_the_reference(dtype, sizes):
    heads, rank, rot, page = sizes['heads'], sizes['rank'], sizes['rot'], sizes['page']
    g = torch.Generator().manual_seed(heads)
    n_tokens = 150
    order = torch.randperm(-(-n_tokens // page) + 2, generator=g).tolist()
    latent, rope, table, _, _ = paged(n_tokens, page, rank, rot, dtype, g, order)
    positions = torch.tensor([0, 1, page - 1, page, page + 1, 63, 64, 65, 127, 128, 149], dtype=torch.int32)
    n = len(positions)
    q = torch.randn(n, heads * (rank + rot), generator=g) * 0.5
    sink = torch.randn(heads, generator=g)
    tables = torch.stack([table, torch.zeros_like(table)])                    # a second sequence nobody asks for
    row_seq = torch.zeros(n, dtype=torch.int32)
    for s in (sink, None):
        common = dict(page_size=page, scale=0.3, heads=heads, rank=rank, rot=rot)
        want = refs.latent_attention(q, latent=latent, rope=rope, block_tables=tables, row_seq=row_seq, positions=positions,
                                     sink=s, **common)
        got = ops.latent_attention(q.cuda(), latent=latent.cuda(), rope=rope.cuda(), block_tables=tables.cuda(),
                                   row_seq=row_seq.cuda(), positions=positions.cuda(), sink=None if s is None else s.cuda(),
                                   **common)
        close(got, want, torch.float32, 1.0 if dtype == torch.float32 else 50.0)


@pytest.mark.parametrize('dtype', DTYPES)
def test_one_key_wins_wherever_it_lies_and_the_sink_weighs(dtype):
    """The query points at one key among 700 with a score far above the others: the result is that key's latent, for a
    key far back, on both sides of page borders and of the kernel's tiles of keys, and the newest one; a key one place
    beyond the row's position is not seen.  A sink far above every score leaves nothing, one far below changes nothing."""
    g = torch.Generator().manual_seed(9)
    heads, rank, rot, page, n_tokens = 3, 24, 8, 16, 700
    order = torch.randperm(-(-n_tokens // page), generator=g).tolist()
    latent, rope, table, c, r = paged(n_tokens, page, rank, rot, dtype, g, order)
    keys = torch.cat([c, r], dim=1).float()
    position = 600
    targets = [0, 1, 15, 16, 17, 31, 32, 63, 64, 65, 300, 599, 600]
    rows = []
    for target in targets + [601]:
        rows.append((keys[target] * 60 / keys[target].square().sum()).repeat(heads))      # score 60 for the key itself
    q = torch.stack(rows)
    n = len(rows)
    args = dict(latent=latent.cuda(), rope=rope.cuda(), page_size=page, block_tables=table[None].cuda(),
                row_seq=torch.zeros(n, dtype=torch.int32).cuda(), positions=torch.full((n,), position, dtype=torch.int32).cuda(),
                scale=1.0, heads=heads, rank=rank, rot=rot)
    got = ops.latent_attention(q.cuda(), sink=None, **args).cpu().view(n, heads, rank)
    others = (q.view(n, heads, -1)[:, 0] @ keys[:position + 1].t())                    # [n, keys]
    for i, target in enumerate(targets):
        rival = others[i][torch.arange(position + 1) != target].max().item()
        assert rival < 45, 'the inputs must let one key stand out'
        torch.testing.assert_close(got[i], c[target].float().expand(heads, rank), atol=1e-3, rtol=1e-3)
    assert (got[-1] - c[601].float()).abs().max() > 0.5                                # not visible yet: not what comes out
    high = ops.latent_attention(q.cuda(), sink=torch.full((heads,), 100.0).cuda(), **args).cpu()
    assert high[:len(targets)].abs().max() < 1e-6
    low = ops.latent_attention(q.cuda(), sink=torch.full((heads,), -80.0).cuda(), **args).cpu().view(n, heads, rank)
    torch.testing.assert_close(low, got, atol=1e-6, rtol=1e-6)
    level = ops.latent_attention(q.cuda(), sink=torch.tensor([60.0, -80.0, 100.0]).cuda(), **args).cpu().view(n, heads, rank)
    torch.testing.assert_close(level[0, 0], 0.5 * c[targets[0]].float(), atol=1e-3, rtol=1e-3)   # a sink level with the winner: half


def scan_inputs(dtype, g, *, n, heads, dim, vdim):
    proj = torch.randn(n, 2 * heads * dim + 2 * heads * vdim, generator=g).to(dtype)
    return proj, dict(heads=heads, dim=dim, vdim=vdim, q_offset=0, k_offset=heads * dim, v_offset=2 * heads * dim)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('mode', ['decay', 'mlstm'])
@pytest.mark.parametrize('sizes', [dict(heads=2, dim=24, vdim=16, rot=8), dict(heads=3, dim=72, vdim=130, rot=72),
                                   dict(heads=1, dim=200, vdim=64, rot=0), dict(heads=2, dim=5, vdim=3, rot=2)])
@pytest.mark.parametrize('steps', [pytest.param((([4, 1, 9], [7, 0, 0]), ([1, 6, 2], [11, 1, 9])), id='token-by-token'),
                                   pytest.param((([130, 1, 64], [7, 0, 0]), ([65, 200, 2], [137, 1, 64])), id='blocks')])
def test_state_scan_against_the_reference(dtype, mode, sizes, steps):
    """Three sequences in one step (one continues from a state, two begin; slots out of order and one used before),
    then a second step that continues all of them with other lengths.  With long sequences the step runs in blocks of
    tokens side by side: whole blocks, a block of one token, sequences that end inside a block."""
    heads, dim, vdim, rot = sizes['heads'], sizes['dim'], sizes['vdim'], sizes['rot']
    g = torch.Generator().manual_seed(dim)
    slot = ops.state_scan_slot(heads=heads, dim=dim, vdim=vdim, mode=mode)
    assert slot == refs.state_scan_slot(heads=heads, dim=dim, vdim=vdim, mode=mode)
    state_c = torch.randn(5, slot, generator=g)
    if mode == 'mlstm':                                            # every block's copy of the maximum alike
        tiles, mats = -(-vdim // 16), heads * dim * vdim
        tops = state_c[:, mats + heads * dim:].view(5, heads, tiles + 1)
        tops[:] = tops[:, :, :1].clone()
    state_g = state_c.clone().cuda()
    freq = torch.tensor([50.0 ** (-2 * i / max(rot, 2)) for i in range(rot // 2)], dtype=torch.float32)
    extra_c = dict(frequencies=freq if rot else None, rot=rot, q_scale=dim ** -0.5, k_scale=0.7)
    if mode == 'mlstm':
        bias = torch.randn(2 * heads, generator=g)
        extra_c.update(gate_bias=bias, cap=6.0)
    else:
        extra_c.update(decay=torch.tensor([0.9, 0.99, 0.999][:heads]))
    for counts, starts in steps:
        n = sum(counts)
        assert (max(counts) >= ops.SCAN_BLOCKS_FROM) == (max(counts) > 9)
        proj, where = scan_inputs(dtype, g, n=n, heads=heads, dim=dim, vdim=vdim)
        cu = torch.tensor([0] + torch.tensor(counts).cumsum(0).tolist(), dtype=torch.int32)
        st, sl = torch.tensor(starts, dtype=torch.int32), torch.tensor([3, 0, 4], dtype=torch.int32)
        step_c = dict(extra_c)
        if mode == 'mlstm':
            step_c['gates'] = torch.randn(n, 2 * heads, generator=g) * 3
        step_g = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in step_c.items()}
        want = refs.state_scan(proj, mode=mode, state=state_c, cu_seqlens=cu, seq_starts=st, seq_slots=sl, n_seqs=3,
                               **where, **step_c)
        got = ops.state_scan(proj.cuda(), mode=mode, state=state_g, cu_seqlens=cu.cuda(), seq_starts=st.cuda(),
                             seq_slots=sl.cuda(), n_seqs=3, max_query=max(counts), **where, **step_g)
        close(got[0], want[0], torch.float32, max(1.0, want[0].abs().max().item()))
        if mode == 'mlstm':
            close(got[1], want[1], torch.float32, max(1.0, want[1].abs().max().item()))
        else:
            assert got[1] is None
        close(state_g[[0, 3, 4]], state_c[[0, 3, 4]], torch.float32, max(1.0, state_c[[0, 3, 4]].abs().max().item()))
        assert torch.equal(state_g[[1, 2]].cpu(), state_c[[1, 2]])               # nobody's slots are left alone


def test_a_decaying_state_remembers_the_first_token_and_forgets_by_its_decay():
    """One value written at the first token, nothing afterwards: what a later query reads is decay**distance of it,
    through steps of any size, and a second sequence in another slot reads nothing of it."""
    heads, dim, vdim = 2, 8, 4
    decay = torch.tensor([0.5, 0.999])
    state = torch.full((3, ops.state_scan_slot(heads=heads, dim=dim, vdim=vdim, mode='decay')), float('nan')).cuda()
    where = dict(heads=heads, dim=dim, vdim=vdim, q_offset=0, k_offset=heads * dim, v_offset=2 * heads * dim, mode='decay',
                 state=state, decay=decay.cuda())

    def rows(n, first):
        proj = torch.zeros(n, 2 * heads * dim + 2 * heads * vdim)
        proj[:, :heads * dim] = 1.0                                             # every query reads every state row
        if first:
            proj[0, heads * dim:2 * heads * dim] = 1.0 / dim                    # key of the first token: sums to 1 under the query
            proj[0, 2 * heads * dim:2 * heads * dim + heads * vdim] = 3.0
        return proj.cuda()

    seen, at = [], 0
    for n in (1, 2, 5, 1, 30):
        cu, st, sl = (torch.tensor(v, dtype=torch.int32).cuda() for v in ([0, n, n + 2], [at, 0], [2, 0]))
        out = ops.state_scan(torch.cat([rows(n, at == 0), rows(2, False)]), cu_seqlens=cu, seq_starts=st, seq_slots=sl,
                             n_seqs=2, **where)[0].cpu()
        seen.append(out[:n])
        assert out[n:].abs().max() == 0                                         # the other sequence begins empty, each time
        at += n
    seen = torch.cat(seen).view(at, heads, vdim)
    distance = torch.arange(at, dtype=torch.float64)
    for h in range(heads):
        want = (3.0 * decay[h].double() ** distance).float()
        torch.testing.assert_close(seen[:, h, 0], want, atol=1e-6, rtol=2e-5)


@pytest.mark.parametrize('dtype', DTYPES)
def test_head_norm_and_gate(dtype):
    g = torch.Generator().manual_seed(4)
    n, heads, vdim = 6, 3, 21
    o = torch.randn(n, heads * vdim, generator=g) * 5
    source = torch.randn(n, 10 + heads * vdim, generator=g).to(dtype)
    weight = 1 + 0.3 * torch.randn(heads * vdim, generator=g)
    below = torch.rand(n, heads, generator=g) + 0.1
    for gate, w, b in (('sigmoid', weight, below), ('silu', None, None)):
        got = ops.head_norm_gate(o.cuda(), source.cuda(), gate_offset=10, heads=heads, vdim=vdim,
                                 weight=None if w is None else w.cuda(), eps=1e-5, gate=gate, out_dtype=dtype,
                                 denominators=None if b is None else b.cuda())
        close(got, refs.head_norm_gate(o, source, gate_offset=10, heads=heads, vdim=vdim, weight=w, eps=1e-5, gate=gate,
                                       out_dtype=dtype, denominators=b), dtype, 3.0)


@pytest.mark.parametrize('sizes', [dict(heads=5, rank=32, rot=8, page=4), dict(heads=7, rank=192, rot=40, page=16),
                                   dict(heads=3, rank=400, rot=48, page=8),
                                   dict(heads=16, rank=512, rot=64, page=16), dict(heads=70, rank=48, rot=16, page=8),
                                   dict(heads=40, rank=512, rot=64, page=32)])
@pytest.mark.parametrize('step', ['portions', 'single rows', 'both'])
@pytest.mark.parametrize('key_parts', [None, (64, 1), (32, 3)])
def test_latent_attention_on_the_matrix_cores(sizes, step, key_parts, monkeypatch):
    """bfloat16 caches with the step's description: sequences of several rows (tiles of rows that share staged keys,
    starting at any position), rows alone in their sequences, the keys in one piece and in parts."""
    heads, rank, rot, page = sizes['heads'], sizes['rank'], sizes['rot'], sizes['page']
    g = torch.Generator().manual_seed(rank + heads)
    lengths = {'portions': [(130, 41), (0, 67), (63, 2)], 'single rows': [(200, 1), (0, 1), (64, 1), (31, 1)],
               'both': [(95, 33), (17, 3), (150, 1), (0, 1)]}[step]                # (tokens cached before, rows of the step)
    most = max(a + b for a, b in lengths)
    pages_each = -(-most // page)
    order = torch.randperm(pages_each * len(lengths) + 2, generator=g)
    latent = torch.full((len(order), page, rank), float('nan')).to(torch.bfloat16)
    rope = torch.full((len(order), page, rot), float('nan')).to(torch.bfloat16)
    tables = order[:pages_each * len(lengths)].view(len(lengths), pages_each).to(torch.int32)
    positions, row_seq, cu = [], [], [0]
    for s, (cached, rows) in enumerate(lengths):
        keys = torch.arange(cached + rows)
        slots = tables[s].long()[keys // page] * page + keys % page
        latent.view(-1, rank)[slots] = torch.randn(len(keys), rank, generator=g).to(torch.bfloat16)
        rope.view(-1, rot)[slots] = torch.randn(len(keys), rot, generator=g).to(torch.bfloat16)
        positions += list(range(cached, cached + rows))
        row_seq += [s] * rows
        cu.append(cu[-1] + rows)
    n = len(positions)
    positions, row_seq, cu = (torch.tensor(v, dtype=torch.int32) for v in (positions, row_seq, cu))
    starts = torch.tensor([a for a, _ in lengths], dtype=torch.int32)
    q = torch.randn(n, heads * (rank + rot), generator=g) * 0.4
    sink = torch.randn(heads, generator=g)
    monkeypatch.setattr(ops, 'LATENT_KEY_PARTS', key_parts)
    for s in (sink, None):
        common = dict(page_size=page, scale=(rank + rot) ** -0.5 * 3, heads=heads, rank=rank, rot=rot)
        want = refs.latent_attention(q, latent=latent, rope=rope, block_tables=tables, row_seq=row_seq, positions=positions,
                                     sink=s, **common)
        got = ops.latent_attention(q.cuda(), latent=latent.cuda(), rope=rope.cuda(), block_tables=tables.cuda(),
                                   row_seq=row_seq.cuda(), positions=positions.cuda(), sink=None if s is None else s.cuda(),
                                   cu_seqlens=cu.cuda(), seq_starts=starts.cuda(), n_seqs=len(lengths),
                                   max_query=max(b for _, b in lengths), max_context=most, **common)
        assert torch.isfinite(got).all()
        torch.testing.assert_close(got.cpu(), want, atol=2e-2, rtol=2e-2)          # queries and probabilities are rounded to bfloat16
