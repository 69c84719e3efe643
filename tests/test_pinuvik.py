"""Pinuvik through the engine against the float64 oracle in
tests/oracles/pinuvik_oracle.py: every mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal batches,
recycled pages and slots, window/chunk edges, first tokens, long decoding,
odd sizes, and greedy generation through the scheduler.

The same cases run on the CPU ops (always) and on the HIP kernels (gpu
marker)."""

import copy
import json
import math
import os

import pytest
import torch

from fusioninfer_amd.config import CacheConfig, EngineConfig, SchedulerConfig
from fusioninfer_amd.engine.llm_engine import LLMEngine
from fusioninfer_amd.engine.sequence import SamplingParams
from fusioninfer_amd.models import registry
from fusioninfer_amd.ops import seqmix
from tests.oracles import pinuvik_oracle as oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def layer_cfg(heads=4, kv_heads=2, dim=24, rot=16, chunk=7, scale=0.3,
              rheads=3, rdim=16, ff=40, base=500.0, rank=5):
    return {
        "type": "parallel",
        "mixer": {
            "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                     "vdim": dim, "scale": scale,
                     "mask": {"size": chunk},
                     "rot": {"dims": rot, "base": base}},
            "right": {"heads": rheads, "dim": rdim, "decay_rank": rank},
        },
        "mlp": {"kind": "dense", "ff": ff} if ff else None,
    }


def small_config():
    """Sizes chosen so that nothing coincides: grouped kv heads, partial
    rotary, a chunk that is neither a power of two nor a multiple of the
    page size, layers that differ, one layer without MLP, a loop that
    starts after the first layer."""
    return {
        "architecture": "Pinuvik",
        "vocab": 97,
        "width": 48,
        "norm": {"eps": 1e-3},
        "loop": {"start": 1, "stop": 3, "times": 2},
        "layers": [
            layer_cfg(),
            layer_cfg(heads=2, kv_heads=1, dim=32, rot=32, chunk=19,
                      scale=0.11, rheads=2, rdim=24, ff=0, rank=3),
            layer_cfg(heads=3, kv_heads=3, dim=16, rot=0, chunk=5,
                      scale=0.5, rheads=1, rdim=40, ff=56, rank=8),
            layer_cfg(heads=6, kv_heads=2, dim=8, rot=6, chunk=64,
                      scale=1.0, rheads=4, rdim=8, ff=24, rank=2),
        ],
    }


def make_engine(raw, device, dtype="float32", blocks=64, max_seqs=4,
                seed=0, budget=4096, eager=True):
    mc = registry.model_config_from_dict(raw)
    mc.dtype = dtype
    cfg = EngineConfig(
        model=mc,
        cache=CacheConfig(num_gpu_blocks=blocks, enable_prefix_caching=False),
        scheduler=SchedulerConfig(max_num_seqs=max_seqs,
                                  max_num_batched_tokens=budget,
                                  max_model_len=blocks * 16,
                                  prefill_admission_tokens=0),
        enforce_eager=eager,
        num_state_slots=max_seqs,
        seed=seed,
    )
    eng = LLMEngine(cfg, device=device)
    model = eng.runner.model
    model.randomize_small_params(seed + 1)
    # livelier weights than the 0.02-std init so that every branch matters
    g = torch.Generator().manual_seed(seed + 2)
    for name, p in model.named_parameters():
        if p.dim() == 2:
            p.data.copy_((torch.randn(p.shape, generator=g)
                          / math.sqrt(p.shape[1])).to(p.dtype).to(p.device))
    W = {k: v.detach().cpu().to(torch.float64)
         for k, v in model.export_weights().items()}
    return eng, W


def rel_err(got, want):
    """Mean-free RMS difference relative to the RMS of the expected row."""
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()).max().item()


def run_schedule(eng, steps):
    """steps: [[(id, tokens, want)], ...] with ('end', id) tuples allowed;
    returns {id: {position: logits}}."""
    got, at = {}, {}
    for step in steps:
        entries = [e for e in step if e[0] != "end"]
        end = [e[1] for e in step if e[0] == "end"]
        out = eng.forced_step(entries, end)
        row = 0
        for rid, toks, want in entries:
            for w in want:
                got.setdefault(rid, {})[at.get(rid, 0) + w] = out[row]
                row += 1
            at[rid] = at.get(rid, 0) + len(toks)
        for rid in end:
            at.pop(rid, None)
    return got


def tokens(n, seed, vocab=97):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


TOL = 2e-4   # fp32 engine vs float64 oracle, relative


# ------------------------------------------------------------ mechanisms
@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_and_scalar_norm(device):
    torch.manual_seed(0)
    W_, T = 40, 9
    x = torch.randn(T, W_)
    mix = torch.rand(W_)
    g = torch.tensor([1.7])
    h = oracle.scalar_norm(x.double(), 1.7, 1e-3)
    want_a = oracle.token_shift(h[:4], mix.double())
    want_b = oracle.token_shift(h[4:], mix.double(), h_before=h[3])
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    state = torch.full((3, W_), 7.0, device=device)   # stale slot content
    a = seqmix.norm_token_shift(x[:4].to(device), g.to(device),
                                mix.to(device), state, mk([0, 4]),
                                mk([0] * 4), mk([0, 1, 2, 3]), mk([2]), 1e-3,
                                torch.float32)
    b = seqmix.norm_token_shift(x[4:].to(device), g.to(device),
                                mix.to(device), state, mk([0, 5]),
                                mk([0] * 5), mk([4, 5, 6, 7, 8]), mk([2]),
                                1e-3, torch.float32)
    assert (a.cpu().double() - want_a).abs().max() < 1e-5
    assert (b.cpu().double() - want_b).abs().max() < 1e-5
    n = seqmix.scalar_rms_norm(x.to(device), g.to(device), 1e-3,
                               torch.float32)
    assert (n.cpu().double() - h).abs().max() < 1e-5


def _attention_case(device, dim, rot, chunk, T, H=2, G=1, pos0=0, seed=0,
                    boost=None, decode_tail=0):
    """Product attention (cache write + ranged attention) on one sequence
    fed as two portions, against the oracle's whole-sequence attention.
    boost=(i, j): query i and key j get one large shared direction so the
    score (i, j) dominates row i if and only if j is visible."""
    torch.manual_seed(seed)
    width = 32
    m = {"heads": H, "kv_heads": G, "dim": dim, "vdim": dim, "scale": 0.4,
         "mask": {"size": chunk}, "rot": {"dims": rot, "base": 100.0}}
    Wq = torch.randn(H * dim, width, dtype=torch.float64) / 6
    Wk = torch.randn(G * dim, width, dtype=torch.float64) / 6
    Wo = torch.eye(H * dim, dtype=torch.float64)
    h = torch.randn(T, width, dtype=torch.float64)
    if boost is not None:
        i, j = boost
        h[i] = h[i] * 0.05
        h[j] = h[j] * 0.05
        # rows i and j share one strong hidden direction
        d = torch.randn(width, dtype=torch.float64)
        h[i] += 4 * d
        h[j] += 4 * d
    want = oracle.shared_kv_attention(
        h, {"q": Wq, "k": Wk, "o": Wo}, "", m, 1e-3)
    from fusioninfer_amd.models.mixers import rotary_inv_freq

    bs, nb = 16, (T + 15) // 16 + 2
    kc = torch.zeros(nb, G, bs, dim, device=device)
    vc = torch.zeros_like(kc)
    blocks = list(range(nb - 1, 0, -1))[: (T + 15) // 16]   # non-identity
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    bt = mk([blocks])
    inv = rotary_inv_freq(rot, 100.0).to(device)
    q = (h @ Wq.T).float().to(device)
    k = (h @ Wk.T).float().to(device)
    outs = []
    cut = T // 2 + 1
    spans = [(0, cut), (cut, T - decode_tail)]
    spans += [(t, t + 1) for t in range(T - decode_tail, T)]  # one by one
    for a, b in spans:
        if b <= a:
            continue
        pos = list(range(a, b))
        slots = [blocks[p // bs] * bs + p % bs for p in pos]
        qn = seqmix.rope_unitnorm_cache_(q[a:b], k[a:b], mk(pos), inv, 1e-3,
                                         kc, vc, mk(slots), H, G, dim)
        outs.append(seqmix.ranged_paged_attention(
            qn.view(b - a, H, dim), kc, vc, bt, mk([0] * (b - a)), mk(pos),
            0.4, chunk=chunk, seq_cu=mk([0, b - a]),
            tiles=(seqmix.build_attention_tiles([b - a], device=device)
                   if b - a > 1 else None)))
    got = torch.cat(outs).reshape(T, H * dim).cpu().double()
    return got, want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dim,rot,chunk", [(16, 16, 6), (24, 10, 17),
                                           (32, 0, 200), (8, 8, 1)])
def test_shared_kv_attention_matches_oracle(device, dim, rot, chunk):
    got, want = _attention_case(device, dim, rot, chunk, T=45)
    assert (got - want).abs().max() < 2e-5


@pytest.mark.parametrize("device", DEVICES)
def test_chunk_edge_one_key_in_or_out(device):
    """chunk = 20: row 39 must see key 20 (first of its chunk) and must
    not see key 19; row 40 starts a chunk and sees only itself."""
    for boost in [(39, 20), (39, 19), (40, 39), (59, 40), (59, 39)]:
        got, want = _attention_case(device, 16, 16, 20, T=64, boost=boost,
                                    seed=boost[0] + boost[1])
        assert (got - want).abs().max() < 2e-5, boost


@pytest.mark.parametrize("device", DEVICES)
def test_chunk_edge_while_decoding(device):
    """Same edges with the last rows fed one token at a time: the decode
    row that opens a chunk sees only itself, the next one sees exactly
    two keys, and a row deep in a chunk still finds the chunk's first
    key but not the key before it."""
    for boost in [(40, 39), (41, 40), (41, 39), (59, 40), (59, 39)]:
        got, want = _attention_case(device, 16, 16, 20, T=60, boost=boost,
                                    seed=3 + boost[0] + boost[1],
                                    decode_tail=22)
        assert (got - want).abs().max() < 2e-5, boost


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds(device):
    """One early key shares the last row's direction: with a chunk as
    long as the sequence it must dominate, across many pages."""
    got, want = _attention_case(device, 16, 8, 1000, T=300, boost=(299, 3),
                                seed=5)
    assert (got - want).abs().max() < 2e-5
    # and for a decoded row (last 5 rows one by one)
    got, want = _attention_case(device, 16, 8, 1000, T=300, boost=(299, 3),
                                seed=6, decode_tail=5)
    assert (got - want).abs().max() < 2e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,dim", [(2, 12), (1, 40)])
def test_delta_rule_matches_oracle_and_carries_state(device, heads, dim):
    torch.manual_seed(3)
    width, T, n = 20, 14, heads * dim
    m = {"heads": heads, "dim": dim}
    names = ["r", "k", "v", "g", "a"]
    W = {x: torch.randn(n, width, dtype=torch.float64) / 3 for x in names}
    W["w1"] = torch.randn(4, width, dtype=torch.float64) / 3
    W["w2"] = torch.randn(n, 4, dtype=torch.float64)
    W["w0"] = torch.randn(n, dtype=torch.float64)
    W["a.b"] = torch.randn(n, dtype=torch.float64)
    W["norm"] = torch.rand(n, dtype=torch.float64) + 0.5
    W["o"] = torch.eye(n, dtype=torch.float64)
    h = torch.randn(T, width, dtype=torch.float64)
    want, S_want = oracle.delta_rule_mixer(h, W, "", m, 1e-3)
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    f = lambda t: t.float().to(device)
    state = torch.full((2, heads, dim, dim), 3.0, device=device)  # stale
    outs = []
    for a, b in ((0, 1), (1, 9), (9, 10), (10, 14)):
        hh = h[a:b]
        wlin = torch.tanh(hh @ W["w1"].T) @ W["w2"].T
        outs.append(seqmix.delta_rule(
            f(hh @ W["r"].T), f(hh @ W["k"].T), f(hh @ W["v"].T), f(wlin),
            f(hh @ W["a"].T), f(hh @ W["g"].T), f(W["w0"]), f(W["a.b"]),
            f(W["norm"]), state, mk([0, b - a]), mk([1]),
            mk(list(range(a, b))), heads, dim, 1e-3, math.exp(-0.5)))
    got = torch.cat(outs).cpu().double()
    assert (got - want).abs().max() < 5e-5
    assert (state[1].cpu().double() - S_want).abs().max() < 5e-5
    assert torch.all(state[0] == 3.0)


@pytest.mark.parametrize("device", DEVICES)
def test_gelu_gate(device):
    torch.manual_seed(4)
    gu = torch.randn(5, 2 * 37) * 3
    want = oracle.gelu_tanh(gu[:, :37].double()) * gu[:, 37:].double()
    got = seqmix.gelu_tanh_and_mul(gu.to(device)).cpu().double()
    assert (got - want).abs().max() < 1e-5


# ----------------------------------------------------- model through engine
@pytest.fixture(scope="module", params=DEVICES)
def small(request):
    raw = small_config()
    eng, W = make_engine(raw, request.param)
    toks = tokens(70, 11)
    want = oracle.forward(raw, W, toks)
    return raw, eng, W, toks, want


def test_layer_streams_and_logits_whole_prompt(small):
    raw, eng, W, toks, want = small
    got = run_schedule(eng, [[("a", toks, list(range(len(toks))))],
                             [("end", "a")]])
    rows = torch.stack([got["a"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL
    # the first tokens of a sequence on their own
    assert rel_err(rows[:3], want[:3]) < TOL


def test_prefill_against_token_by_token_decoding(small):
    raw, eng, W, toks, want = small
    steps = [[("d", toks[:1], [0])]]
    steps += [[("d", [t], [0])] for t in toks[1:]]
    steps.append([("end", "d")])
    got = run_schedule(eng, steps)
    rows = torch.stack([got["d"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL


@pytest.mark.parametrize("sizes", [[2] * 35, [3, 16, 1, 2, 31, 2, 15],
                                   [33, 2, 35], [64, 2, 2, 2]])
def test_portions_of_several_sizes(small, sizes):
    raw, eng, W, toks, want = small
    assert sum(sizes) == len(toks)
    steps, a = [], 0
    for n in sizes:
        steps.append([("p", toks[a:a + n], list(range(n)))])
        a += n
    steps.append([("end", "p")])
    got = run_schedule(eng, steps)
    rows = torch.stack([got["p"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL


def test_unequal_batch_equals_each_alone_and_recycles(small):
    raw, eng, W, toks, want = small
    reqs = {"r0": tokens(41, 1), "r1": tokens(5, 2), "r2": tokens(23, 3),
            "r3": tokens(1, 4), "r4": tokens(37, 5), "r5": tokens(18, 6)}
    ref = {k: oracle.forward(raw, W, v) for k, v in reqs.items()}
    all_ = lambda n: list(range(n))
    t = reqs
    steps = [
        [("r0", t["r0"][:7], all_(7)), ("r1", t["r1"][:2], all_(2))],
        [("r0", t["r0"][7:8], [0]), ("r1", t["r1"][2:], all_(3)),
         ("r2", t["r2"][:20], all_(20)), ("r3", t["r3"], [0]),
         ("end", "r1"), ("end", "r3")],
        # r4 and r5 take the slots and pages r1 and r3 gave back
        [("r4", t["r4"][:30], all_(30)), ("r0", t["r0"][8:9], [0]),
         ("r5", t["r5"][:1], [0]), ("r2", t["r2"][20:21], [0])],
        [("r5", t["r5"][1:2], [0]), ("r0", t["r0"][9:41], all_(32)),
         ("r2", t["r2"][21:], all_(2)), ("r4", t["r4"][30:31], [0]),
         ("end", "r0"), ("end", "r2")],
        [("r4", t["r4"][31:], all_(6)), ("r5", t["r5"][2:], all_(16)),
         ("end", "r4"), ("end", "r5")],
    ]
    free_before = (eng.block_manager.num_free(), eng.state_manager.num_free())
    got = run_schedule(eng, steps)
    for k, v in reqs.items():
        rows = torch.stack([got[k][p] for p in range(len(v))])
        assert rel_err(rows, ref[k]) < TOL, k
    assert (eng.block_manager.num_free(),
            eng.state_manager.num_free()) == free_before


def test_slot_and_pages_reused_by_a_shorter_request(small):
    """A long request leaves state and pages behind; the next one in the
    same slot and pages must start from nothing."""
    raw, eng, W, toks, want = small
    run_schedule(eng, [[("x", tokens(60, 9), [])], [("end", "x")]])
    got = run_schedule(eng, [[("y", toks[:9], list(range(9)))],
                             [("end", "y")]])
    rows = torch.stack([got["y"][p] for p in range(9)])
    assert rel_err(rows, want[:9]) < TOL


def test_greedy_generation_through_scheduler(small):
    raw, eng, W, toks, want = small
    prompts = [toks[:13], toks[20:23], toks[30:51]]
    n_new = 12
    outs = eng.generate(prompts, SamplingParams(max_tokens=n_new))
    for p, o in zip(prompts, outs):
        assert o.output_token_ids == oracle.greedy(raw, W, p, n_new)
    assert eng.state_manager.num_free() == eng.state_manager.num_slots


def test_generation_with_small_token_budget_chunks_prompts():
    """The scheduler's own chunked prefill (budget 8 tokens a step) and
    more requests than slots."""
    raw = small_config()
    eng, W = make_engine(raw, "cpu", max_seqs=2, budget=8, seed=3)
    prompts = [tokens(21, 31), tokens(9, 32), tokens(14, 33)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=6))
    for p, o in zip(prompts, outs):
        assert o.output_token_ids == oracle.greedy(raw, W, p, 6)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_across_chunks_and_pages(device):
    raw = {
        "architecture": "Pinuvik", "vocab": 50, "width": 32,
        "norm": {"eps": 1e-5}, "loop": {"start": 0, "stop": 1, "times": 3},
        "layers": [layer_cfg(heads=2, kv_heads=2, dim=16, rot=16, chunk=24,
                             scale=0.25, rheads=2, rdim=16, ff=32)],
    }
    eng, W = make_engine(raw, device, blocks=16)
    toks = tokens(150, 21, vocab=50)
    want = oracle.forward(raw, W, toks)
    steps = [[("a", toks[:10], list(range(10)))]]
    steps += [[("a", [t], [0])] for t in toks[10:]]
    got = run_schedule(eng, steps)
    rows = torch.stack([got["a"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL


@pytest.mark.parametrize("device", DEVICES)
def test_values_that_could_hide_faults(device):
    """heads == kv_heads == 1, full rotary, chunk 1 (every token alone),
    loop run once, single layer without MLP."""
    raw = {
        "architecture": "Pinuvik", "vocab": 31, "width": 16,
        "norm": {"eps": 1e-6}, "loop": {"start": 0, "stop": 0, "times": 5},
        "layers": [layer_cfg(heads=1, kv_heads=1, dim=8, rot=8, chunk=1,
                             scale=2.0, rheads=1, rdim=4, ff=0, rank=1)],
    }
    eng, W = make_engine(raw, device, blocks=8)
    toks = tokens(20, 7, vocab=31)
    want = oracle.forward(raw, W, toks)
    got = run_schedule(eng, [[("a", toks[:11], list(range(11)))],
                             [("a", toks[11:], list(range(9)))]])
    rows = torch.stack([got["a"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL


def test_checkpoint_directory_roundtrip(tmp_path):
    """config.json + model.safetensors -> registry -> engine: sizes that
    the config does not carry come from tensor shapes; bf16 storage."""
    from safetensors.torch import save_file

    raw = small_config()
    eng, W = make_engine(raw, "cpu", dtype="bfloat16")
    disk = {k: v.to(torch.bfloat16) for k, v in
            eng.runner.model.export_weights().items()}
    cfg_disk = copy.deepcopy(raw)
    for L in cfg_disk["layers"]:
        del L["mixer"]["right"]["decay_rank"]
    d = tmp_path / "m"
    os.makedirs(d)
    save_file(disk, str(d / "model.safetensors"))
    (d / "config.json").write_text(json.dumps(cfg_disk))
    mc = registry.get_model_config(str(d))
    assert mc.architecture == "Pinuvik"
    assert [L.right.decay_rank for L in mc.arch.layers] == [5, 3, 8, 2]
    mc.dtype = "float32"
    cfg = EngineConfig(model=mc, cache=CacheConfig(num_gpu_blocks=16),
                       scheduler=SchedulerConfig(max_num_seqs=2,
                                                 max_model_len=256),
                       enforce_eager=True)
    eng2 = LLMEngine(cfg, device="cpu")
    W2 = {k: v.to(torch.float64) for k, v in disk.items()}
    toks = tokens(25, 8)
    want = oracle.forward(cfg_disk, W2, toks)
    got = run_schedule(eng2, [[("a", toks, list(range(25)))]])
    rows = torch.stack([got["a"][p] for p in range(25)])
    assert rel_err(rows, want) < TOL
    with pytest.raises(ValueError):
        eng2.runner.model.load_weights([("embed", disk["embed"])])


def test_bf16_mode_stays_close_to_oracle():
    raw = small_config()
    eng, W = make_engine(raw, "cpu", dtype="bfloat16")
    toks = tokens(40, 12)
    want = oracle.forward(raw, W, toks)
    got = run_schedule(eng, [[("a", toks[:30], list(range(30)))],
                             [("a", toks[30:], list(range(10)))]])
    rows = torch.stack([got["a"][p] for p in range(40)])
    assert rel_err(rows, want) < 0.08


def test_state_slot_manager_and_scheduler_limits():
    from fusioninfer_amd.engine.sequence import Sequence
    from fusioninfer_amd.engine.state_manager import StateSlotManager

    sm = StateSlotManager(2)
    a, b, c = (Sequence(n, [1], SamplingParams()) for n in "abc")
    assert sm.allocate(a) == 0 and sm.allocate(b) == 1
    assert not sm.can_allocate()
    with pytest.raises(RuntimeError):
        sm.allocate(c)
    sm.free(a)
    assert a.state_slot == -1 and sm.allocate(c) == 0
    sm.free(a)  # freeing twice is a no-op
    assert sm.num_free() == 0


@pytest.mark.gpu
def test_hipgraph_decode_replays_match_oracle():
    """All-decode steps replay captured graphs (batch buckets 1, 2, 4);
    replays alternate with eager prefill portions and with steps of other
    batch sizes, and every replay is compared with the oracle."""
    raw = small_config()
    eng, W = make_engine(raw, "cuda", eager=False, blocks=48)
    assert eng.runner._graphs, "decode graphs were not captured"
    reqs = {k: tokens(n, s) for k, n, s in
            [("a", 30, 1), ("b", 26, 2), ("c", 22, 3)]}
    ref = {k: oracle.forward(raw, W, v) for k, v in reqs.items()}
    t = reqs
    steps = [[("a", t["a"][:8], list(range(8)))],
             [("b", t["b"][:5], list(range(5))), ("a", t["a"][8:9], [0])]]
    for i in range(9, 20):          # graph replays, batch 2
        steps.append([("a", t["a"][i:i + 1], [0]),
                      ("b", t["b"][i - 4:i - 3], [0])])
    steps.append([("c", t["c"][:12], list(range(12)))])   # eager between
    for i in range(20, 30):         # graph replays, batch 3 -> bucket 4
        steps.append([("a", t["a"][i:i + 1], [0]),
                      ("b", t["b"][i - 4:i - 3], [0]),
                      ("c", t["c"][i - 8:i - 7], [0])])
    got = run_schedule(eng, steps)
    for k in reqs:
        ps = sorted(got[k])
        rows = torch.stack([got[k][p] for p in ps])
        assert rel_err(rows, ref[k][ps]) < TOL, k


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_engine_matches_cpu_engine_at_larger_sizes(dtype):
    """Head sizes with tiled kernels (128, 64), grouped kv heads, partial
    rotary, chunks that straddle tiles and pages, a few hundred tokens:
    the HIP path against the CPU ops on identical weights, through
    portions, decoding and a mixed batch."""
    raw = {
        "architecture": "Pinuvik", "vocab": 211, "width": 192,
        "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 2, "times": 2},
        "layers": [
            layer_cfg(heads=4, kv_heads=2, dim=128, rot=64, chunk=150,
                      scale=0.09, rheads=2, rdim=128, ff=320, rank=12),
            layer_cfg(heads=6, kv_heads=3, dim=64, rot=64, chunk=97,
                      scale=0.125, rheads=3, rdim=64, ff=0, rank=7),
        ],
    }
    cpu, W = make_engine(raw, "cpu", dtype=dtype, blocks=96, seed=5)
    gpu, W2 = make_engine(raw, "cuda", dtype=dtype, blocks=96, seed=5)
    for k in W:
        assert torch.equal(W[k], W2[k]), k
    a, b = tokens(420, 41, vocab=211), tokens(333, 42, vocab=211)
    every = lambda n, step=7: list(range(0, n, step))
    steps = [
        [("a", a[:300], every(300))],
        [("a", a[300:301], [0]), ("b", b[:131], every(131))],
        [("a", a[301:302], [0]), ("b", b[131:133], [0, 1])],
        [("a", a[302:420], every(118)), ("b", b[133:134], [0])],
    ]
    steps += [[("b", [t], [0])] for t in b[134:170]]
    steps += [[("b", b[170:], every(163, 5)), ("end", "a")], [("end", "b")]]
    want = run_schedule(cpu, steps)
    got = run_schedule(gpu, steps)
    lim = 2e-4 if dtype == "float32" else 0.05
    for rid in want:
        ps = sorted(want[rid])
        assert sorted(got[rid]) == ps
        e = rel_err(torch.stack([got[rid][p] for p in ps]),
                    torch.stack([want[rid][p] for p in ps]))
        assert e < lim, (rid, e)


def test_forced_steps_serve_the_transformer_family_too():
    """forced_step is the engine's own batch path: on the built-in
    transformer its logits reproduce what greedy generation picks."""
    mc = registry.get_model_config("tiny-qwen3")
    cfg = EngineConfig(model=mc, cache=CacheConfig(num_gpu_blocks=64),
                       scheduler=SchedulerConfig(max_num_seqs=4,
                                                 max_model_len=512),
                       enforce_eager=True, seed=3)
    eng = LLMEngine(cfg, device="cpu")
    prompt = tokens(19, 77, vocab=1000)
    out = eng.generate([prompt], SamplingParams(max_tokens=5))[0]
    toks = prompt + out.output_token_ids
    # prompt in two portions, then the generated tokens one at a time
    lg = [eng.forced_step([("x", toks[:11], [])]),
          eng.forced_step([("x", toks[11:19], [7])])]
    picked = [int(lg[1][0].argmax())]
    for i in range(19, 23):
        picked.append(int(eng.forced_step([("x", [toks[i]], [0])])[0]
                          .argmax()))
    eng.forced_step([], ["x"])
    assert picked == out.output_token_ids
    assert eng.block_manager.num_free() == 64


@pytest.mark.gpu
def test_generation_with_graph_replay_and_pipelined_decode():
    """engine.generate on the GPU with captured decode graphs: admission,
    chunked prefill, graph replays fed by on-device sampled ids, slot
    recycling (more prompts than slots) - token-exact with the oracle."""
    raw = small_config()
    eng, W = make_engine(raw, "cuda", eager=False, max_seqs=2, budget=16,
                         seed=9)
    assert eng.runner._graphs
    prompts = [tokens(21, 51), tokens(5, 52), tokens(33, 53), tokens(2, 54)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10))
    for p, o in zip(prompts, outs):
        assert o.output_token_ids == oracle.greedy(raw, W, p, 10)
    assert eng.state_manager.num_free() == 2
