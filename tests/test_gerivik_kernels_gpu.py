"""The kernels behind the Gerivik design, each alone against its plain reference (``kernel_refs``) on the same inputs, in
float32 and bfloat16, at sizes that are no multiples of anything; and inputs made so that one fault shows: a router
whose correction and groups decide, an expert that every token or no token chooses, identity experts, a cap that
saturates, a decay of almost nothing and of almost everything."""
import math

import pytest
import torch

import kernel_refs as refs
from qil_amd import ops
from qil_amd.parts.base import Rotation
from test_kernels_gpu import build_cache

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def close(actual, expected, dtype, scale=1.0):
    tolerance = dict(atol=2e-5 * scale, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2 * scale, rtol=2e-2)
    torch.testing.assert_close(actual.float().cpu(), expected.float(), **tolerance)


def test_embedding_with_a_scale():
    g = torch.Generator().manual_seed(0)
    for dtype, width in ((torch.float32, 20), (torch.bfloat16, 24), (torch.bfloat16, 21)):
        table = torch.randn(11, width, generator=g).to(dtype)
        tokens = torch.tensor([3, 0, 10, 3], dtype=torch.int32)
        got = ops.embed(tokens.cuda(), table.cuda(), 12.5)
        assert torch.equal(got.cpu(), table[tokens.long()].float() * 12.5)


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('width', [40, 257, 1100, 5000])
def test_a_normed_output_joins_the_stream_under_the_next_norm(dtype, width):
    g = torch.Generator().manual_seed(width)
    n = 7
    stream = torch.randn(n, width, generator=g) * 3 + 1.5
    weight, post = 1 + 0.1 * torch.randn(width, generator=g), 1 + 0.3 * torch.randn(width, generator=g)
    delta = (torch.randn(n, width, generator=g) * 20).to(dtype)
    whole = torch.randn(n, width, generator=g) * 0.01
    parts = torch.randn(3, n, width, generator=g)
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
    for d_gpu, d_cpu in ((delta.cuda(), delta), (ops.Partials(parts.cuda()), parts.sum(0)), (whole.cuda(), whole)):
        s_gpu, s_cpu = stream.clone().cuda(), stream.clone()
        got = ops.add_rmsnorm(s_gpu, ops.PostNormed(d_gpu, post.cuda(), 1e-5), weight.cuda(), 1e-6, dtype)
        want = refs.add_rmsnorm(s_cpu, ops.PostNormed(d_cpu, post, 1e-5), weight, 1e-6, dtype)
        close(got, want, dtype)
        close(s_gpu, s_cpu, torch.float32)                                     # the stream holds the unrounded sum
        expected = stream + d_cpu.float() / torch.sqrt(d_cpu.float().square().mean(-1, keepdim=True) + 1e-5) * post
        close(s_gpu, expected, torch.float32)
        before = s_gpu.clone()
        got = ops.rows_rmsnorm(s_gpu, ops.PostNormed(d_gpu, post.cuda(), 1e-5), rows.cuda(), weight.cuda(), 1e-6, dtype)
        close(got, refs.rows_rmsnorm(s_cpu, ops.PostNormed(d_cpu, post, 1e-5), rows, weight, 1e-6, dtype), dtype)
        assert torch.equal(before, s_gpu)


# ------------------------------------------------------------------------------------------------ queries and keys
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('sizes', [dict(heads=4, kv_heads=2, d=64, rot=16), dict(heads=3, kv_heads=1, d=24, rot=6),
                                   dict(heads=2, kv_heads=2, d=128, rot=128), dict(heads=5, kv_heads=5, d=40, rot=2)])
def test_rotation_from_frequencies_before_a_unit_norm(dtype, sizes):
    """Both q/k kernels (eight elements a lane for heads of 16, 32, ... elements; the general one otherwise), with the
    angle made from the position, the norm behind the rotation, and heads padded with zeros whose mean runs over the true
    size."""
    heads, kv_heads, d, rot = sizes['heads'], sizes['kv_heads'], sizes['d'], sizes['rot']
    g = torch.Generator().manual_seed(d)
    n, page = 9, 4
    qkv = torch.randn(n, (heads + 2 * kv_heads) * d, generator=g).to(dtype)
    true_d = d - 4 if d % 16 else d                            # padded heads: zeros behind the true size
    if true_d != d:
        qkv.view(n, heads + 2 * kv_heads, d)[:, :, true_d:] = 0
    frequencies = torch.tensor([300.0 ** (-2 * i / rot) for i in range(rot // 2)], dtype=torch.float32)
    positions = torch.tensor([0, 1, 2, 700, 4, 5, 100000, 7, 8], dtype=torch.int32)
    slots = torch.tensor([4, 5, 6, 7, 0, 1, 2, 3, 9], dtype=torch.int32)
    ones = torch.ones(d)
    caches_c = [torch.zeros(3, kv_heads, page, d, dtype=dtype), torch.zeros(3, kv_heads, d, page, dtype=dtype)]
    caches_g = [c.clone().cuda() for c in caches_c]
    for first in (True, False):
        args = dict(heads=heads, kv_heads=kv_heads, head_dim=d, eps=1e-6, page_size=page, dtype=dtype, norm_dim=true_d,
                    rotate_first=first)
        want = refs.qk_norm_rope_store(qkv, q_weight=ones, k_weight=ones, rotation=Rotation(None, None, rot, frequencies),
                                       positions=positions, slots=slots, k_cache=caches_c[0], v_cache=caches_c[1], **args)
        got = ops.qk_norm_rope_store(qkv.cuda(), q_weight=ones.cuda(), k_weight=ones.cuda(),
                                     rotation=Rotation(None, None, rot, frequencies.cuda()), positions=positions.cuda(),
                                     slots=slots.cuda(), k_cache=caches_g[0], v_cache=caches_g[1], **args)
        close(got, want, dtype)
        close(caches_g[0], caches_c[0], dtype)
        close(caches_g[1], caches_c[1], dtype)
    # a rotation keeps a head's root mean square: with no weights to speak of, the two orders agree to rounding
    unit = got.float().view(n, heads, d).square().sum(-1) / true_d
    close(unit, torch.ones(n, heads), dtype)


# ------------------------------------------------------------------------------------------------ capped attention
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('lengths,page_size,d,heads,kv_heads', [
    ([1, 15, 16, 17], 16, 64, 6, 3),
    ([65, 3, 511, 257], 3, 40, 6, 2),
    ([1025, 1, 256], 16, 128, 4, 1),
    ([300, 2], 4, 48, 5, 5),
])
@pytest.mark.parametrize('cap', [0.5, 30.0])
def test_capped_scores_in_decoding_and_in_prompts(dtype, lengths, page_size, d, heads, kv_heads, cap):
    """Single rows (the split-context kernels) and the last rows of every sequence as a portion (the tile kernel, also
    with its keys in parts) against the reference; a cap of 0.5 saturates nearly every score, which an uncapped kernel
    would not survive."""
    k_cache, v_cache, table, _ = build_cache(lengths, page_size, kv_heads, d, dtype)
    scale = 3.0 * d ** -0.5
    common = dict(heads=heads, kv_heads=kv_heads, head_dim=d, k_cache=k_cache, v_cache=v_cache, page_size=page_size,
                  block_tables=table, scale=scale, window=None, max_context=max(lengths))
    cpu = dict(common, k_cache=k_cache.cpu(), v_cache=v_cache.cpu(), block_tables=table.cpu())
    g = torch.Generator().manual_seed(len(lengths))
    # decoding: one row a sequence
    rows = len(lengths)
    q = torch.randn(rows, heads * d, generator=g).to(dtype)
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
    row_seq = torch.arange(rows, dtype=torch.int32)
    step = dict(cu_seqlens=None, seq_starts=None, single_rows=None, n_seqs=rows, max_query=1)
    got = ops.paged_attention(q.cuda(), row_seq=row_seq.cuda(), positions=positions.cuda(), softcap=cap, **step, **common)
    want = refs.paged_attention(q, row_seq=row_seq, positions=positions, softcap=cap, **step, **cpu)
    close(got, want, dtype)
    uncapped = refs.paged_attention(q, row_seq=row_seq, positions=positions, softcap=None, **step, **cpu)
    assert (want.float() - uncapped.float()).abs().max() > (0.05 if cap < 1 else 0)
    # portions: the last rows of every sequence, sequences of several rows first
    counts = sorted((min(n, 37) for n in lengths), reverse=True)
    order = sorted(range(rows), key=lambda i: -min(lengths[i], 37))
    cu = [0]
    for c in counts:
        cu.append(cu[-1] + c)
    n = cu[-1]
    q = torch.randn(n, heads * d, generator=g).to(dtype)
    starts = [lengths[i] - c for i, c in zip(order, counts)]
    positions = torch.tensor([s + t for s, c in zip(starts, counts) for t in range(c)], dtype=torch.int32)
    row_seq = torch.tensor([i for i, c in enumerate(counts) for _ in range(c)], dtype=torch.int32)
    single = torch.tensor([cu[i] for i, c in enumerate(counts) if c == 1], dtype=torch.int32)
    tables = table[torch.tensor(order).cuda()].contiguous()
    step = dict(n_seqs=rows, max_query=max(counts), tile_seqs=sum(c > 1 for c in counts))
    got = ops.paged_attention(q.cuda(), row_seq=row_seq.cuda(), positions=positions.cuda(), softcap=cap,
                              cu_seqlens=torch.tensor(cu, dtype=torch.int32).cuda(),
                              seq_starts=torch.tensor(starts, dtype=torch.int32).cuda(), single_rows=single.cuda(),
                              **step, **dict(common, block_tables=tables))
    want = refs.paged_attention(q, row_seq=row_seq, positions=positions, softcap=cap, cu_seqlens=None, seq_starts=None,
                                single_rows=None, **step, **dict(cpu, block_tables=tables.cpu()))
    close(got, want, dtype)


@pytest.mark.parametrize('lengths,page_size,d,heads,kv_heads,rot,splits,cap', [
    ([1, 2, 31, 32, 33, 64, 65, 96], 8, 64, 6, 2, 32, 3, 0.5),
    ([2100, 1, 700, 1290, 64, 2047, 300, 33], 16, 128, 16, 4, 64, 8, 30.0),
    ([257, 512, 513], 32, 128, 8, 1, 128, 1, 5.0),
])
def test_decoding_with_queries_made_inside_is_the_two_kernels(lengths, page_size, d, heads, kv_heads, rot, splits, cap):
    """The decode kernel that makes queries, the new key and the new value itself, with the rotation from frequencies
    before a unit norm and capped scores: bit for bit what the q/k kernel followed by the attention kernel leave."""
    dtype = torch.bfloat16
    rows, total = len(lengths), heads + 2 * kv_heads
    k_cache, v_cache, table, _ = build_cache(lengths, page_size, kv_heads, d, dtype)
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32).cuda()
    row_seq = torch.arange(rows, dtype=torch.int32).cuda()
    slots = (table[row_seq.long(), (positions // page_size).long()] * page_size + positions % page_size).to(torch.int32)
    g = torch.Generator().manual_seed(d)
    qkv = ops.Partials((torch.randn(splits, rows, total * d, generator=g) * 0.7).cuda())
    ones = torch.ones(d).cuda()
    frequencies = torch.tensor([5000.0 ** (-2 * i / rot) for i in range(rot // 2)], dtype=torch.float32).cuda()
    rotation = Rotation(None, None, rot, frequencies)
    sizes = dict(heads=heads, kv_heads=kv_heads, head_dim=d)
    assert ops.decode_attention_takes(qkv, page_size=page_size, rotation=rotation, dtype=dtype, **sizes)
    k_two, v_two = k_cache.clone(), v_cache.clone()
    q = ops.qk_norm_rope_store(qkv, q_weight=ones, k_weight=ones, eps=1e-6, rotation=rotation, positions=positions,
                               slots=slots, k_cache=k_two, v_cache=v_two, page_size=page_size, dtype=dtype,
                               rotate_first=True, **sizes)
    want = ops.paged_attention(q, k_cache=k_two, v_cache=v_two, page_size=page_size, block_tables=table, row_seq=row_seq,
                               positions=positions, cu_seqlens=None, seq_starts=None, single_rows=None, n_seqs=rows,
                               max_query=1, max_context=max(lengths), scale=2.0 * d ** -0.5, window=None, softcap=cap, **sizes)
    k_one, v_one = k_cache.clone(), v_cache.clone()
    got = ops.decode_attention(qkv, q_weight=ones, k_weight=ones, eps=1e-6, rotation=rotation, positions=positions,
                               writes=True, k_cache=k_one, v_cache=v_one, page_size=page_size, block_tables=table,
                               row_seq=row_seq, max_context=max(lengths), scale=2.0 * d ** -0.5, window=None,
                               rotate_first=True, softcap=cap, **sizes)
    assert torch.isfinite(got.float()).all()
    torch.testing.assert_close(got, want, atol=0, rtol=0)
    same = lambda a, b: torch.equal(a.view(torch.int16), b.view(torch.int16))          # NaN-filled pages: compare the bits
    assert same(k_one, k_two) and same(v_one, v_two), 'the pages differ'
    uncapped = ops.decode_attention(qkv, q_weight=ones, k_weight=ones, eps=1e-6, rotation=rotation, positions=positions,
                                    writes=False, k_cache=k_one, v_cache=v_one, page_size=page_size, block_tables=table,
                                    row_seq=row_seq, max_context=max(lengths), scale=2.0 * d ** -0.5, window=None,
                                    rotate_first=True, softcap=None, **sizes)
    assert not torch.equal(uncapped, got)


# ------------------------------------------------------------------------------------------------ the memory's decays
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('sizes', [dict(heads=2, dim=24, vdim=16), dict(heads=3, dim=72, vdim=130),
                                   dict(heads=1, dim=200, vdim=64), dict(heads=2, dim=5, vdim=3)])
@pytest.mark.parametrize('steps', [pytest.param((([4, 1, 9], [7, 0, 0]), ([1, 6, 2], [11, 1, 9])), id='token-by-token'),
                                   pytest.param((([130, 1, 64], [7, 0, 0]), ([65, 200, 2], [137, 1, 64])), id='blocks')])
def test_a_decay_for_every_row_of_the_memory(dtype, sizes, steps):
    """Three sequences in one step (one continues from a state, two begin; slots out of order), then a second step that
    continues all of them; token by token and in blocks of 64 tokens, with decay logits from -12 (a row forgets at
    once) to 12 (it keeps everything) and a tau that sharpens them."""
    heads, dim, vdim = sizes['heads'], sizes['dim'], sizes['vdim']
    g = torch.Generator().manual_seed(dim)
    slot = ops.state_scan_slot(heads=heads, dim=dim, vdim=vdim, mode='channel')
    assert slot == heads * dim * vdim == refs.state_scan_slot(heads=heads, dim=dim, vdim=vdim, mode='channel')
    state_c = torch.randn(5, slot, generator=g)
    state_g = state_c.clone().cuda()
    where = dict(heads=heads, dim=dim, vdim=vdim, q_offset=0, k_offset=heads * dim, v_offset=2 * heads * dim)
    for counts, starts in steps:
        n = sum(counts)
        proj = torch.randn(n, 2 * heads * dim + 2 * heads * vdim, generator=g).to(dtype)
        z = torch.randn(n, heads * dim, generator=g) * 4
        z[:, 0], z[:, -1] = -12.0, 12.0
        cu = torch.tensor([0] + torch.tensor(counts).cumsum(0).tolist(), dtype=torch.int32)
        st, sl = torch.tensor(starts, dtype=torch.int32), torch.tensor([3, 0, 4], dtype=torch.int32)
        extra = dict(cap=0.75, q_scale=dim ** -0.5, k_scale=1.0)
        want = refs.state_scan(proj, mode='channel', state=state_c, cu_seqlens=cu, seq_starts=st, seq_slots=sl, n_seqs=3,
                               gates=z, **where, **extra)
        got = ops.state_scan(proj.cuda(), mode='channel', state=state_g, cu_seqlens=cu.cuda(), seq_starts=st.cuda(),
                             seq_slots=sl.cuda(), n_seqs=3, max_query=max(counts), gates=z.cuda(), **where, **extra)
        assert got[1] is None
        close(got[0], want[0], torch.float32, max(1.0, want[0].abs().max().item()))
        close(state_g[[0, 3, 4]], state_c[[0, 3, 4]], torch.float32, max(1.0, state_c[[0, 3, 4]].abs().max().item()))
        assert torch.equal(state_g[[1, 2]].cpu(), state_c[[1, 2]])               # nobody's slots are left alone


def test_a_row_forgets_by_its_own_decay():
    """One value written at the first token, nothing afterwards: what a later query reads through row i of the memory
    is a_i ** distance of it, in steps of any size (single tokens, short runs, blocks)."""
    heads, dim, vdim, tau = 1, 8, 4, 2.0
    z = torch.linspace(-3.0, 6.0, dim)
    keep = torch.sigmoid(z) ** (1 / tau)
    total = 300
    proj = torch.zeros(total, 2 * dim + 2 * vdim)
    proj[0, dim:2 * dim] = 1.0                                   # the first key writes into every row
    proj[0, 2 * dim:2 * dim + vdim] = torch.tensor([1.0, -2.0, 3.0, 0.5])
    for t in range(total):
        proj[t, t % dim] = 1.0                                   # query t reads row t % dim
    state = torch.full((2, dim * vdim), float('nan')).cuda()
    outs, at = [], 0
    for size in (1, 1, 5, 70, 1, 64, 130, 28):
        got, _ = ops.state_scan(proj[at:at + size].cuda(), mode='channel', heads=heads, dim=dim, vdim=vdim, q_offset=0,
                                k_offset=dim, v_offset=2 * dim, state=state,
                                cu_seqlens=torch.tensor([0, size], dtype=torch.int32).cuda(),
                                seq_starts=torch.tensor([at], dtype=torch.int32).cuda(),
                                seq_slots=torch.tensor([1], dtype=torch.int32).cuda(), n_seqs=1, max_query=size,
                                gates=z.repeat(size, 1).cuda(), cap=tau)
        outs.append(got.cpu())
        at += size
    got = torch.cat(outs)
    for t in (0, 1, 7, 8, 77, 141, 299):
        expected = keep[t % dim].double() ** t * proj[0, 2 * dim:2 * dim + vdim].double()
        torch.testing.assert_close(got[t].double(), expected, atol=1e-6, rtol=2e-4)


# ------------------------------------------------------------------------------------------------ the routed feed-forward
@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('sizes', [dict(width=40, outputs=18, groups=3, keep=2, top=4), dict(width=256, outputs=64, groups=8, keep=3, top=6),
                                   dict(width=33, outputs=5, groups=1, keep=1, top=5), dict(width=64, outputs=130, groups=10, keep=10, top=1),
                                   dict(width=24, outputs=9, groups=9, keep=2, top=2)])
def test_the_router_against_the_reference(dtype, sizes):
    g = torch.Generator().manual_seed(sizes['outputs'])
    n, width, outputs = 50, sizes['width'], sizes['outputs']
    x = torch.randn(n, width, generator=g).to(dtype)
    router = torch.randn(outputs, width, generator=g) * 0.4
    correction = torch.randn(outputs, generator=g) * 0.3 - 1.0          # negative choice scores: dropped groups are -inf, not 0
    rule = dict(groups=sizes['groups'], keep=sizes['keep'], top=sizes['top'])
    for c_gpu, c_cpu, renormalize in ((correction.cuda(), correction, False), (None, None, True)):
        chosen, weights = ops.moe_route(x.cuda(), router.cuda(), c_gpu, renormalize=renormalize, **rule)
        want_chosen, want_weights = refs.moe_route(x, router, c_cpu, renormalize=renormalize, **rule)
        assert torch.equal(chosen.cpu().sort(dim=1).values, want_chosen.sort(dim=1).values)
        assert torch.equal(chosen.cpu(), want_chosen)                   # best first, as the reference orders them
        close(weights, want_weights, torch.float32)
        if renormalize:
            close(weights.sum(dim=1), torch.ones(n), torch.float32)


def test_the_router_by_hand():
    """Six outputs in three groups of which two are kept: the correction moves the choice and not the weights; a group
    goes by its best corrected score; what is outside the kept groups is out however good it is."""
    width = 8
    logit = torch.tensor([2.0, 0.0, 1.9, 1.8, 0.5, 0.4])
    x = torch.zeros(1, width)
    x[0, 0] = 1.0
    router = torch.zeros(6, width)
    router[:, 0] = logit
    s = torch.softmax(logit, dim=0)
    rule = dict(groups=3, keep=2, top=2)
    chosen, weights = ops.moe_route(x.cuda(), router.cuda(), torch.zeros(6).cuda(), **rule)
    assert chosen.tolist() == [[0, 2]] and torch.allclose(weights.cpu()[0], s[[0, 2]])
    chosen, weights = ops.moe_route(x.cuda(), router.cuda(), torch.tensor([0.0, 0.0, 0.0, 0.0, 0.9, 0.0]).cuda(), **rule)
    assert chosen.tolist() == [[4, 0]] and torch.allclose(weights.cpu()[0], s[[4, 0]])
    chosen, _ = ops.moe_route(x.cuda(), router.cuda(), torch.tensor([-5.0, -5.0, -5.0, -5.0, -5.0, -5.1]).cuda(), **rule)
    assert chosen.tolist() == [[0, 2]]


@pytest.mark.parametrize('dtype', DTYPES)
@pytest.mark.parametrize('sizes', [dict(n=5, width=40, ff=16, experts=6, identity=2, top=3),
                                   dict(n=300, width=64, ff=48, experts=3, identity=0, top=2),       # tiles of 64 pairs
                                   dict(n=260, width=200, ff=144, experts=2, identity=1, top=2),    # stages of 64 columns with a rest
                                   dict(n=70, width=36, ff=32, experts=4, identity=4, top=4),        # width no multiple of 8
                                   dict(n=1, width=192, ff=96, experts=10, identity=1, top=2),
                                   dict(n=33, width=136, ff=80, experts=1, identity=1, top=2)])
def test_the_experts_against_the_reference(dtype, sizes):
    g = torch.Generator().manual_seed(sizes['width'])
    n, width, ff, experts, top = sizes['n'], sizes['width'], sizes['ff'], sizes['experts'], sizes['top']
    outputs = experts + sizes['identity']
    x = torch.randn(n, width, generator=g).to(dtype)
    gate_up = (torch.randn(experts, 2, ff, width, generator=g) * 2 / math.sqrt(width)).to(dtype)
    down = (torch.randn(experts, width, ff, generator=g) / math.sqrt(ff)).to(dtype)
    chosen = torch.stack([torch.randperm(outputs, generator=g)[:top] for _ in range(n)]).to(torch.int32)
    weights = torch.rand(n, top, generator=g)
    if n > 3:
        chosen[1], chosen[2] = torch.arange(top), torch.arange(outputs - top, outputs)     # the first and the last outputs
    act = dict(activation='clamped_swish', limit=1.0, alpha=1.702)
    got = ops.moe_experts(x.cuda(), chosen.cuda(), weights.cuda(), gate_up.cuda(), down.cuda(), **act)
    want = refs.moe_experts(x, chosen, weights, gate_up, down, **act)
    close(got, want, dtype, max(1.0, want.abs().max().item()))
    # left for the next norm to sum: the same numbers through the norm's kernel as through the sum's own
    lazy = ops.moe_experts(x.cuda(), chosen.cuda(), weights.cuda(), gate_up.cuda(), down.cuda(), lazy=True, **act)
    close(lazy.materialize(), want, dtype, max(1.0, want.abs().max().item()))
    stream, post, weight = torch.randn(n, width, generator=g), 1 + 0.1 * torch.randn(width, generator=g), torch.ones(width)
    through = [s.clone().cuda() for s in (stream, stream)]
    one = ops.add_rmsnorm(through[0], ops.PostNormed(lazy, post.cuda(), 1e-6), weight.cuda(), 1e-6, dtype)
    two = ops.add_rmsnorm(through[1], ops.PostNormed(got, post.cuda(), 1e-6), weight.cuda(), 1e-6, dtype)
    close(through[0], through[1].cpu(), torch.float32)
    close(one, two.cpu(), dtype)
    # a token's result does not depend on who else is in the step
    alone = ops.moe_experts(x[:1].cuda(), chosen[:1].cuda(), weights[:1].cuda(), gate_up.cuda(), down.cuda(), **act)
    assert torch.equal(alone[0], got[0])


def test_the_routed_part_against_experts_one_by_one():
    from qil_amd.parts import RoutedExperts
    g = torch.Generator().manual_seed(2)
    width, ff, n = 24, 20, 12                                      # ff is padded to 32 inside the part
    part = RoutedExperts(width=width, experts=3, identity=1, top=2, groups=2, keep=1, intermediate=ff,
                         activation='clamped_swish', limit=0.8, alpha=1.702, correction=True, dtype=torch.float32)
    tensors = {name: torch.randn(spec.shape, generator=g) * (0.5 if 'proj' in name else 1.0) for name, spec in part.param_specs().items()}
    for name, t in tensors.items():
        part.set_param(name, t.cuda())
    part.finalize()
    h = torch.randn(n, width, generator=g)
    out = part.forward(h.cuda()).materialize().cpu()
    s = torch.softmax(h @ tensors['router.weight'].t(), dim=-1)
    choice = s + tensors['router.correction']
    group = choice.view(n, 2, 2).max(-1).values.argmax(-1)
    for row in range(n):
        pair = [2 * int(group[row]), 2 * int(group[row]) + 1]
        expected = torch.zeros(width)
        for e in pair:
            if e == 3:
                expected += s[row, e] * h[row]
                continue
            a = (tensors[f'experts.{e}.gate_proj.weight'] @ h[row]).clamp(max=0.8)
            b = (tensors[f'experts.{e}.up_proj.weight'] @ h[row]).clamp(-0.8, 0.8)
            expected += s[row, e] * (tensors[f'experts.{e}.down_proj.weight'] @ (a * torch.sigmoid(1.702 * a) * (b + 1)))
        torch.testing.assert_close(out[row], expected, atol=2e-5, rtol=2e-5)
