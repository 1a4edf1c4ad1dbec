"""The Fubapel design in the engine against its plain whole-sequence restatement (``plain_fubapel``), under every way
of cutting the work: whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, pages and
state slots that are freed and used again, and generation through the serving loop.

Each test runs three ways, as the step function's own tests do: on the CPU with the kernels' plain references
substituted (block tables, slots, state slots, row selection, the schedule with repeated layers), and on the GPU with
the HIP kernels in float32 and in bfloat16 (marked ``gpu``).  Page and state storage is filled with NaN first.
Configurations are small and their sizes differ from one another in every field (heads, head sizes, ranks, rotated
widths, numbers of state columns above and below one wave, repeated spans in different places).
"""
import json
import random

import pytest
import torch

import plain_fubapel as plain
from conftest import write_model_folder
from qil_amd.engine import ModelRunner, StepEntry
from qil_amd.weights import load_model

BACKENDS = [pytest.param(('cpu', torch.float32), id='cpu-refs'),
            pytest.param(('cuda', torch.float32), id='gpu-f32', marks=pytest.mark.gpu),
            pytest.param(('cuda', torch.bfloat16), id='gpu-bf16', marks=pytest.mark.gpu)]

# every mixer once, one of them repeated; a feed-forward on some layers only
MIXED = plain.make_config(
    [plain.attention_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=24, ff=80, limit=1.0),
     plain.mlstm_layer(heads=2, dim=24, vdim=16, gate_cap=15.0),
     plain.retention_layer(heads=3, dim=16, vdim=24, decay=(0.9, 0.97, 0.995), rot_dims=8, ff=64, limit=0.75),
     plain.attention_layer(heads=1, dim=8, rot_dim=4, vdim=8, kv_rank=12, q_rank=10)],
    vocab=97, width=48, loop=dict(start=1, stop=3, times=2), residual_mult=0.8)
# the recurrent layers repeated, state columns beyond one wave (80, 130), sizes that are no powers of two
WIDE = plain.make_config(
    [plain.mlstm_layer(heads=2, dim=40, vdim=80, gate_cap=8.0, ff=56, limit=1.5),
     plain.retention_layer(heads=2, dim=72, vdim=130, decay=(0.95, 0.999), rot_dims=72),
     plain.attention_layer(heads=5, dim=12, rot_dim=6, vdim=10, kv_rank=20, q_rank=14, base=300.0)],
    vocab=61, width=40, loop=dict(start=0, stop=2, times=3), residual_mult=1.0)
# attention alone, repeated; nothing else
ATTENTION = plain.make_config(
    [plain.attention_layer(heads=4, dim=24, rot_dim=16, vdim=8, kv_rank=32, q_rank=16, ff=48, limit=2.5)],
    vocab=50, width=32, loop=dict(start=0, stop=1, times=2), residual_mult=0.5)
# (configuration, seed, page size, spread of the matrices: smaller where repeated recurrent layers amplify roundings)
CONFIGS = {'mixed': (MIXED, 11, 8, 0.25), 'wide': (WIDE, 12, 16, 0.25), 'attention': (ATTENTION, 13, 4, 1.0)}


def tokens_for(config, length, seed):
    r = random.Random(seed)
    return [r.randrange(config['vocab']) for _ in range(length)]


def error(actual, expected):
    """The largest row error: root mean square over the vocabulary of the difference (its mean taken off), over the
    root mean square of the expected logits."""
    difference = actual.double().cpu() - expected.double()
    difference = difference - difference.mean(dim=-1, keepdim=True)
    return (difference.square().mean(dim=-1).sqrt() / expected.double().square().mean().sqrt()).max().item()


# The plain model itself, run in float32, is 3e-7 to 2e-5 from float64 on these configurations, and run with every
# operation rounded to bfloat16 0.01 to 0.04; the engine in bfloat16 (activations between kernels rounded; state,
# gates, norms and sums float32) 0.01 to 0.045.  A sequence that loses its context half way (a lost state, another
# request's pages) is 0.08 to 0.6 away.
LIMIT = {torch.float32: 1e-4, torch.bfloat16: 0.06}


class Case:
    def __init__(self, name, config, weights, model, page_size, dtype):
        self.name, self.config, self.weights, self.model, self.page_size, self.dtype = name, config, weights, model, page_size, dtype
        self._expected = {}

    def expected(self, tokens):
        key = tuple(tokens)
        if key not in self._expected:
            self._expected[key] = plain.logits(tokens, self.weights, self.config)
        return self._expected[key]

    def runner(self, pages, requests=4, graphs=False):
        runner = ModelRunner(self.model, num_pages=pages, page_size=self.page_size, max_requests=requests, graphs=graphs)
        for group in runner.cache.kv_groups:
            for tensor in group['tensors'].values():
                tensor.fill_(float('nan'))
        for group in runner.cache.state_groups:
            group['state'].fill_(float('nan'))
        return runner

    def close(self, actual, expected, what=''):
        assert torch.isfinite(actual).all(), what
        e = error(actual, expected)
        assert e <= LIMIT[self.dtype], f'{what}: error {e:.3e} ({self.dtype})'


@pytest.fixture(params=BACKENDS)
def backend(request):
    device, dtype = request.param
    if device == 'cpu':
        request.getfixturevalue('cpu_kernels')
    return device, dtype


@pytest.fixture(params=sorted(CONFIGS))
def case(request, backend, tmp_path):
    device, dtype = backend
    config, seed, page_size, spread = CONFIGS[request.param]
    weights = plain.random_weights(config, seed, spread)
    folder = write_model_folder(tmp_path / request.param, config, weights, torch.bfloat16)
    return Case(request.param, config, weights, load_model(folder, dtype=dtype, device=device), page_size, dtype)


def feed(runner, name, tokens, cuts, want_all=True):
    """One request alone, its tokens in steps of the given sizes (the rest one by one); the logits of every place."""
    runner.admit(name)
    rows, at, sizes = [], 0, list(cuts)
    while at < len(tokens):
        size = min(sizes.pop(0) if sizes else 1, len(tokens) - at)
        rows.append(runner.step([StepEntry(name, tuple(tokens[at:at + size]), tuple(range(size)))]))
        at += size
    runner.release(name)
    return torch.cat(rows)


def test_whole_prompts(case):
    runner = case.runner(pages=64)
    for length, seed in ((1, 1), (2, 2), (37, 3), (150, 4)):
        tokens = tokens_for(case.config, length, seed)
        case.close(feed(runner, 'r', tokens, [length]), case.expected(tokens), f'{length} tokens')
    runner.cache.check()


def test_decoding_token_by_token_equals_the_prompt(case):
    """The first tokens of a sequence one by one, then a long run of single tokens behind a prompt."""
    runner = case.runner(pages=64)
    tokens = tokens_for(case.config, 45, 5)
    case.close(feed(runner, 'r', tokens, []), case.expected(tokens), 'one by one from the first token')
    tokens = tokens_for(case.config, 140, 6)
    case.close(feed(runner, 'r', tokens, [50]), case.expected(tokens), '50, then 90 single tokens')


def test_decode_graphs_replay_the_same_logits(case):
    if case.model.device.type != 'cuda':
        pytest.skip('graphs are a GPU matter')
    runner = case.runner(pages=64, graphs=True)
    tokens = tokens_for(case.config, 70, 7)
    case.close(feed(runner, 'r', tokens, [20]), case.expected(tokens), 'decode steps from graphs')
    assert runner.graphs.safe() and runner.graphs.replays >= 20


@pytest.mark.parametrize('cuts', [[2] * 40, [3, 2, 17, 2, 5, 31, 2, 2, 9], [16, 16, 1, 15, 33, 7], [63, 2, 1, 1, 2]])
def test_portions_of_changing_size(case, cuts):
    """Portions down to two tokens, cut inside pages and at their borders; the rest token by token."""
    runner = case.runner(pages=64)
    tokens = tokens_for(case.config, 90, 8)
    case.close(feed(runner, 'r', tokens, cuts), case.expected(tokens), f'cuts {cuts[:6]}')


def test_unequal_requests_together_and_slots_used_again(case):
    """Up to three live requests of unequal lengths, portions beside single tokens; requests end and others take their
    pages and state slots (three slots, six requests); some steps leave a live request out."""
    lengths = dict(a=71, b=9, c=38, d=1, e=55, f=20)
    sequences = {name: tokens_for(case.config, n, 20 + i) for i, (name, n) in enumerate(lengths.items())}
    pages = -(-(71 + 55 + 38) // case.page_size) + 3
    runner = case.runner(pages=pages, requests=3)
    waiting, live = list(sequences), []
    fed = {name: 0 for name in sequences}
    got = {name: [] for name in sequences}
    r, step = random.Random(3), 0
    used_slots = []
    while waiting or live:
        while waiting and len(live) < 3:
            name = waiting.pop(0)
            assert runner.admit(name)
            used_slots.append(runner.cache.slots[name])
            live.append(name)
        entries = []
        for name in live:
            if len(live) > 1 and r.random() < 0.2:
                continue                                      # left out of this step
            left = len(sequences[name]) - fed[name]
            size = min(left, r.choice([1, 1, 2, 3, 7, 16, 29]))
            entries.append(StepEntry(name, tuple(sequences[name][fed[name]:fed[name] + size]), tuple(range(size))))
        if not entries:
            continue
        logits = runner.step(entries)
        at = 0
        for entry in entries:
            size = len(entry.tokens)
            got[entry.request].append(logits[at:at + size])
            at += size
            fed[entry.request] += size
            if fed[entry.request] == len(sequences[entry.request]):
                runner.release(entry.request)
                live.remove(entry.request)
        runner.cache.check()
        step += 1
    assert sorted(set(used_slots)) == [0, 1, 2] and len(used_slots) == 6
    assert runner.cache.free_pages == [pages] * len(runner.cache.kv_groups)
    for name, tokens in sequences.items():
        case.close(torch.cat(got[name]), case.expected(tokens), f'request {name}')


def test_a_batch_changes_nothing(case):
    """The same request alone and beside others gives the same logits (beyond rounding: the same kernels may split
    their sums differently)."""
    a, b, c = (tokens_for(case.config, n, 40 + n) for n in (33, 12, 50))
    alone = feed(case.runner(pages=32), 'a', a, [20, 2])
    runner = case.runner(pages=32)
    for name in 'abc':
        runner.admit(name)
    rows = [runner.step([StepEntry('b', tuple(b[:5])), StepEntry('a', tuple(a[:20]), tuple(range(20))), StepEntry('c', tuple(c[:31]))])]
    rows.append(runner.step([StepEntry('a', tuple(a[20:22]), (0, 1)), StepEntry('c', tuple(c[31:32])), StepEntry('b', tuple(b[5:]))])[:2])
    for i in range(22, 33):
        rows.append(runner.step([StepEntry('c', (c[i + 10],)), StepEntry('a', (a[i],), (0,))]))
    together = torch.cat(rows)
    assert error(together, alone.cpu()) <= LIMIT[case.dtype] / 2
    case.close(together, case.expected(a), 'beside others')


def test_generation_through_the_serving_loop(case):
    """Greedy generation by the engine's own entry point and scheduler: every drawn token is (within the dtype's
    rounding) the best one of the plain logits of the engine's own sequence so far."""
    from qil_amd.engine import Engine
    prompts = [tokens_for(case.config, n, 60 + n) for n in (5, 1, 23, 12, 9)]
    engine = Engine(case.model, num_pages=24, page_size=case.page_size, token_budget=20, prefill_chunk=7, max_active=3)
    reports = engine.generate(prompts, max_new_tokens=12, ignore_eos=True)
    engine.cache.check()
    assert engine.cache.free_pages == [24] * len(engine.cache.kv_groups)
    slack = 1e-4 if case.dtype == torch.float32 else 0.05
    for prompt, report in zip(prompts, reports):
        output = report['token_ids']
        assert len(output) == 12 and report['finish_reason'] == 'length'
        rows = plain.logits(prompt + output, case.weights, case.config)
        spread = rows.std().item()
        for index, token in enumerate(output):
            row = rows[len(prompt) + index - 1]
            assert row[token] >= row.max() - slack * spread, f'token {index} of {prompt}'
    if case.dtype == torch.float32:
        assert [r['token_ids'] for r in reports][0] == plain.greedy(prompts[0], 12, case.weights, case.config)


ALONE = {
    'attention-one-head': plain.make_config([plain.attention_layer(heads=1, dim=10, rot_dim=2, vdim=14, kv_rank=9, q_rank=33)],
                                            vocab=40, width=24, residual_mult=1.0),
    'attention-many-heads': plain.make_config([plain.attention_layer(heads=9, dim=4, rot_dim=12, vdim=6, kv_rank=70, q_rank=8,
                                                                     base=20.0, ff=40, limit=0.6)], vocab=40, width=36),
    'gated-memory': plain.make_config([plain.mlstm_layer(heads=3, dim=10, vdim=70, gate_cap=4.0, ff=30, limit=3.0)],
                                      vocab=40, width=30, loop=dict(start=0, stop=1, times=1), residual_mult=0.9),
    'gated-memory-one-head': plain.make_config([plain.mlstm_layer(heads=1, dim=130, vdim=12, gate_cap=30.0)], vocab=40, width=20),
    'decaying-memory': plain.make_config([plain.retention_layer(heads=1, dim=20, vdim=12, decay=(0.8,), rot_dims=20)],
                                         vocab=40, width=16, residual_mult=1.2),
    'decaying-memory-part-rotated': plain.make_config([plain.retention_layer(heads=4, dim=12, vdim=12, decay=(1.0, 0.5, 0.99, 0.9),
                                                                             rot_dims=4, base=7.0, ff=20, limit=1.0)],
                                                      vocab=40, width=28, loop=dict(start=0, stop=1, times=4)),
}


@pytest.mark.parametrize('name', sorted(ALONE))
def test_each_mixer_alone(name, backend, tmp_path):
    """Models of one layer: one mechanism each, at sizes where fields that often coincide differ (head size and value
    size, rank and width, rotated part and head) and where counts are 1."""
    device, dtype = backend
    config = ALONE[name]
    weights = plain.random_weights(config, 5, 0.5)
    folder = write_model_folder(tmp_path / name, config, weights, torch.bfloat16)
    case = Case(name, config, weights, load_model(folder, dtype=dtype, device=device), 8, dtype)
    tokens = tokens_for(config, 60, 9)
    runner = case.runner(pages=16)
    case.close(feed(runner, 'r', tokens, [60]), case.expected(tokens), 'whole')
    case.close(feed(runner, 'r', tokens, [13, 2, 9, 8, 16]), case.expected(tokens), 'portions, then single tokens')


def test_config_round_trip_and_refusals(tmp_path):
    from qil_amd.config import ConfigError, FubapelConfig
    from qil_amd.registry import architecture_for
    typed = FubapelConfig.from_dict(MIXED)
    assert architecture_for(MIXED).name == 'Fubapel' and typed.layer_order() == [0, 1, 2, 1, 2, 3]
    assert FubapelConfig.from_dict(json.loads(json.dumps(typed.to_dict()))) == typed
    assert FubapelConfig.from_dict({k: v for k, v in MIXED.items() if k != 'loop'}).layer_order() == [0, 1, 2, 3]
    for broken in (dict(MIXED, loop=dict(start=2, stop=1, times=1)), dict(MIXED, window=4), dict(MIXED, residual_mult=0),
                   dict(MIXED, layers=[dict(MIXED['layers'][0], type='conv')]),
                   dict(MIXED, layers=[dict(MIXED['layers'][1], mixer=dict(MIXED['layers'][1]['mixer'], window=3))]),
                   dict(MIXED, layers=[dict(MIXED['layers'][2], mixer=dict(MIXED['layers'][2]['mixer'], decay=[0.5]))])):
        with pytest.raises(ConfigError):
            FubapelConfig.from_dict(broken)


def test_the_plain_model_cuts_like_its_parts():
    """The oracle itself: a prefix's logits do not depend on what follows (every mixer is causal), and the layers run
    in the configured order."""
    weights = plain.random_weights(MIXED, 3)
    tokens = tokens_for(MIXED, 30, 1)
    whole, streams = plain.logits(tokens, weights, MIXED), []
    prefix = plain.logits(tokens[:17], weights, MIXED, streams=streams)
    assert torch.allclose(whole[:17], prefix, atol=1e-9) and len(streams) == 6 and plain.layer_order(MIXED) == [0, 1, 2, 1, 2, 3]


@pytest.mark.gpu
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_trace_replay_program(tmp_path, dtype):
    """``bin/trace_run`` on a Fubapel folder: requests alone and whole, their last tokens one by one, portions down to
    two tokens, and up to four live requests in a pool of pages and state slots that is used again."""
    from test_engine_gpu import collect, replay, traces
    config, seed, _, spread = CONFIGS['mixed']
    weights = plain.random_weights(config, seed, spread)
    folder = write_model_folder(tmp_path / 'model', config, weights, torch.bfloat16)
    prompts, shapes = traces(dict(vocab_size=config['vocab']), seed)
    expected = {request: plain.logits(tokens, weights, config) for request, tokens in prompts.items()}
    limit = LIMIT[getattr(torch, dtype)]
    for shape, (steps, max_tokens) in shapes.items():
        out = tmp_path / shape
        replay(folder, dtype, steps, out, max_tokens)
        rows = collect(out, steps, config['vocab'])
        assert rows, shape
        for request, items in rows.items():
            got = torch.stack([row for _, row in items])
            assert torch.isfinite(got).all()
            e = error(got, expected[request][[position for position, _ in items]])
            assert e <= limit, f'{shape} {request}: error {e:.3e}'
