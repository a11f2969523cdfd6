"""Numalorn through the engine (scheduler, latent pages, state slots, kernels or torch ops)
against the slow oracle: whole prompts, decoding, portions, batches, reused pages and slots."""
import pytest
import torch

from . import oracle
from .common import HEAD64, ONLY_WKV, SMALL, alone, build, check, run_schedule, tokens

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [SMALL, HEAD64, ONLY_WKV], ids=["small", "head64", "only_wkv"])
def test_whole_prompt_and_token_by_token(device, cfg):
    eng, full = build(cfg, device)
    t = tokens(70, cfg["vocab"], 1)
    whole = run_schedule(eng, alone(t, []))
    check(whole, cfg, full, {"a": t})
    single = run_schedule(eng, alone(t, [1] * 69))
    check(single, cfg, full, {"a": t})
    mixed = run_schedule(eng, alone(t, [38] + [1] * 32))
    check(mixed, cfg, full, {"a": t})
    assert len(whole) == len(single) == len(mixed) == 70


@pytest.mark.parametrize("device", DEVICES)
def test_layers_one_by_one(device):
    """The residual stream after every layer of a whole prompt."""
    from replisense_rfq_amd.engine.runner import ModelRunner

    cfg = SMALL
    eng, full = build(cfg, device)
    t = tokens(45, cfg["vocab"], 3)
    want = []
    oracle.forward(cfg, full, t, want)
    taps, fwd = [], eng.model.forward
    eng.model.forward = lambda m: fwd(m, taps)
    try:
        run_schedule(eng, alone(t, []))
    finally:
        eng.model.forward = fwd
    assert len(taps) == len(want) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(taps, want)):
        err = float((a.double().cpu() - b).abs().max() / b.abs().max())
        assert err < 1e-4, f"layer {i}: {err:.2e}"
    assert ModelRunner is not None


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[2] * 30, [3, 2, 33, 2, 5, 31, 2], [32, 32, 1, 1, 2], [64, 2],
                                  [7, 7, 7, 7, 7, 7, 7, 7, 7, 7, 2, 1, 1]])
def test_portions(device, cuts):
    """Portions down to two tokens, cut inside pages; short ones run in the decode section
    (<= 32 rows), long ones in the prefill section."""
    eng, full = build(SMALL, device)
    t = tokens(83, SMALL["vocab"], 2)
    check(run_schedule(eng, alone(t, cuts)), SMALL, full, {"a": t})


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_one_token_requests(device):
    eng, full = build(HEAD64, device)
    for n in (1, 2, 3):
        t = tokens(n, HEAD64["vocab"], 10 + n)
        check(run_schedule(eng, alone(t, [])), HEAD64, full, {"a": t})
        check(run_schedule(eng, alone(t, [1] * n)), HEAD64, full, {"a": t})


@pytest.mark.parametrize("device", DEVICES)
def test_batches_of_unequal_requests(device):
    """Up to four live requests, portions beside single tokens, requests that pause, pages and
    slots given back and used again by later requests: each row as if its request ran alone."""
    cfg = SMALL
    eng, full = build(cfg, device, max_kv_blocks=14)       # 13 pages: reuse is forced
    V = cfg["vocab"]
    req = {n: tokens(L, V, 20 + i) for i, (n, L) in enumerate(
        [("a", 97), ("b", 40), ("c", 5), ("d", 66), ("e", 130), ("f", 33), ("g", 64)])}
    at = {n: 0 for n in req}

    def take(n, c):
        lo = at[n]
        at[n] = lo + c
        return (n, req[n][lo:lo + c], list(range(c)))

    plan = [
        [("a", 50), ("b", 2), ("c", 5)], [("a", 1), ("b", 33), ("d", 40)], [("a", 1), ("b", 5)],
        [("a", 45), ("d", 2)], [("d", 24), ("e", 64), ("f", 3)], [("e", 1), ("f", 30)],
        [("e", 2), ("g", 64)], [("e", 63)],
    ]
    steps = []
    for st in plan:
        entries = [take(n, c) for n, c in st]
        steps.append({"entries": entries, "end": [n for n, _ in st if at[n] == len(req[n])]})
    assert all(at[n] == len(req[n]) for n in req)
    got = run_schedule(eng, steps)
    check(got, cfg, full, req)
    assert len(got) == sum(len(t) for t in req.values())
    assert eng.core.num_free_state_slots == 4 and eng.core.num_free_blocks == 13


@pytest.mark.parametrize("device", DEVICES)
def test_slot_and_pages_reused_after_release(device):
    """One slot, pool of one request: each request runs where the last one's state matrices,
    input row and latents still lie."""
    cfg = HEAD64
    eng, full = build(cfg, device, max_num_seqs=1, max_kv_blocks=4)
    for i in range(3):
        t = tokens(70 + i, cfg["vocab"], 40 + i)
        check(run_schedule(eng, alone(t, [33, 2, 1, 1])), cfg, full, {"a": t})


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_over_page_edges(device):
    cfg = SMALL
    eng, full = build(cfg, device)
    t = tokens(140, cfg["vocab"], 50)
    check(run_schedule(eng, alone(t, [20] + [1] * 120)), cfg, full, {"a": t})


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_stands_out(device):
    """One early token whose key every later query of one head is made to match: scaled
    up-projections make its score dominate hundreds of others, in a prompt and in decoding."""
    cfg = SMALL
    _, full = build(cfg, "cpu")
    full = dict(full)
    full["l0.mix.uk"] = full["l0.mix.uk"] * 3.0
    full["l0.mix.sink"] = full["l0.mix.sink"] - 4.0
    eng, _ = build(cfg, device, full=full, max_kv_blocks=40, max_model_len=1024, max_batched_tokens=1024)
    t = tokens(400, cfg["vocab"], 77)
    got = run_schedule(eng, alone(t, [330, 2, 31] + [1] * 37))
    check(got, cfg, full, {"a": t})
    # the strengthened keys matter: the unscaled model's logits differ visibly
    base = oracle.forward(cfg, build(cfg, "cpu")[1], t)
    assert float((base[-1] - got[("a", 399)].double()).abs().max()) > 1e-2


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_close_to_oracle_and_independent_of_cuts(device):
    cfg = SMALL
    eng, full = build(cfg, device, dtype=torch.bfloat16)
    a, b = tokens(100, cfg["vocab"], 80), tokens(41, cfg["vocab"], 81)
    steps = [{"entries": [("a", a[:70], list(range(70))), ("b", b[:3], [0, 1, 2])], "end": []},
             {"entries": [("a", a[70:71], [0]), ("b", b[3:40], list(range(37)))], "end": []},
             {"entries": [("a", a[71:], list(range(29))), ("b", b[40:], [0])], "end": ["a", "b"]}]
    got = run_schedule(eng, steps)
    assert len(got) == 141
    ref = {"a": oracle.forward(cfg, full, a), "b": oracle.forward(cfg, full, b)}

    def err(row, want, std):
        d = row.double() - want.double()
        d = d - d.mean()
        return float(d.pow(2).mean().sqrt() / std)

    # a rounded router input can flip a close choice of experts at a single position: nearly
    # all rows are within rounding of the oracle, and the typical row is far inside
    e = sorted(err(row, ref[n][p], ref[n].std()) for (n, p), row in got.items())
    assert e[len(e) // 2] < 0.03 and e[int(len(e) * 0.95)] < 0.08, (e[len(e) // 2], e[-8:])
    whole = run_schedule(eng, alone(a, []))
    e = sorted(err(whole[("a", p)], got[("a", p)], ref["a"].std()) for p in range(100))
    assert e[50] < 0.03 and e[95] < 0.08, (e[50], e[-8:])


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_engine(device):
    """generate() (scheduler, sampler at temperature 0, decode steps) picks the oracle's tokens."""
    from replisense_rfq_amd.engine.sequence import SamplingParams

    cfg = HEAD64
    eng, full = build(cfg, device)
    prompts = [tokens(n, cfg["vocab"], 70 + n) for n in (9, 35, 2)]
    seqs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, grammar=False))
    for p, s in zip(prompts, seqs):
        assert s.output_ids == oracle.greedy(cfg, full, p, 12)
    assert eng.core.num_free_state_slots == 4


@pytest.mark.parametrize("device", DEVICES)
def test_checkpoint_folder_round_trip(device, tmp_path):
    """config.json + model.safetensors written to a folder choose the model class and load."""
    import json

    from safetensors.torch import save_file

    from replisense_rfq_amd.engine.engine import LLMEngine
    from replisense_rfq_amd.utils.config import EngineConfig

    cfg = ONLY_WKV if device == "cpu" else SMALL
    _, full = build(cfg, "cpu")
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in full.items()},
              str(tmp_path / "model.safetensors"))
    eng = LLMEngine(EngineConfig(model="x", weights_path=str(tmp_path), dtype="float32", device=str(device),
                                 max_num_seqs=2, max_kv_blocks=8, max_batched_tokens=128,
                                 max_model_len=128, use_graphs=False, grammar=False,
                                 prefix_cache=False, warm_prefix=False, tune_gemm=False,
                                 jump_forward=False))
    assert type(eng.model).__name__ == "NumalornLM"
    t = tokens(20, cfg["vocab"], 5)
    check(run_schedule(eng, alone(t, [9, 2])), cfg, full, {"a": t})


@pytest.mark.gpu
def test_layer_sized_model_in_bf16_against_the_torch_ops():
    """Layers of a served model's widths (512-wide cached latent, 128-wide heads, 64-wide
    recurrent heads, experts on the grouped GEMMs), bf16 on the GPU: prompts in portions and
    decoding, against the same weights run in fp32 through the torch ops on the CPU."""
    from .common import latent, moe, wkv, config

    cfg = config([latent(8, 128, 128, 384, 512, 128 ** -0.5, moe(512, 8, 2, 2, 1)),
                  wkv(16, 64, moe(512, 8, 2, 2, 1, 256)),
                  latent(8, 128, 128, 384, 512, 128 ** -0.5, None, kv_from=0)],
                 vocab=1000, width=1024, mult=0.5, cap=30.0)
    kw = dict(max_kv_blocks=40, max_model_len=640, max_batched_tokens=1024)
    ref_eng, full = build(cfg, "cpu", **kw)
    eng, _ = build(cfg, "cuda:0", dtype=torch.bfloat16, full=full, **kw)
    assert all(lw["grouped"] for lw, ly in zip(eng.model.w["layers"], cfg["layers"]) if ly["mlp"])
    a, b = tokens(420, cfg["vocab"], 90), tokens(130, cfg["vocab"], 91)
    steps = [{"entries": [("a", a[:300], [299]), ("b", b[:100], [0, 99])], "end": []},
             {"entries": [("a", a[300:400], [0, 99]), ("b", b[100:101], [0])], "end": []}]
    steps += [{"entries": [("a", a[400 + i:401 + i], [0]), ("b", b[101 + i:102 + i], [0])], "end": []}
              for i in range(20)]
    want = run_schedule(ref_eng, steps)
    got = run_schedule(eng, steps)
    assert len(got) == len(want) == 46
    e = []
    for key, row in got.items():
        d = row.double() - want[key].double()
        d = d - d.mean()
        e.append(float(d.pow(2).mean().sqrt() / want[key].double().std()))
    e.sort()
    assert e[len(e) // 2] < 0.05 and e[-3] < 0.15, e[-6:]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decode_graphs_replayed_between_eager_steps(dtype):
    """Decode steps replay a captured hipGraph (token shift, recurrence, latent attention,
    routing and experts inside it), prompts run eagerly in between: greedy generation of
    several waves of requests picks the oracle's tokens each time (fp32), and the graph was
    the path that ran."""
    from replisense_rfq_amd.engine.sequence import SamplingParams

    cfg = HEAD64
    eng, full = build(cfg, "cuda:0", dtype=dtype, use_graphs=True, graph_buckets=(4,))
    assert eng.runner.graphs
    for wave in range(3):
        prompts = [tokens(n, cfg["vocab"], 100 + 10 * wave + n) for n in (9, 35, 2)]
        seqs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, grammar=False))
        if dtype == torch.float32:
            for p, s in zip(prompts, seqs):
                assert s.output_ids == oracle.greedy(cfg, full, p, 10), wave
    assert eng.runner.stats["graph_steps"] >= 24
    assert eng.core.num_free_state_slots == 4


@pytest.mark.gpu
def test_wide_layers_few_tokens_with_graphs():
    """A 2048-wide layer pair (16 heads of 128 over a 512-wide latent, 32 recurrent heads,
    8 experts of width 4096 on the grouped GEMMs) with decode graphs: a prompt in one eager
    step, then graph steps; finite logits that do not depend on the path (graph or eager)."""
    from replisense_rfq_amd.engine.sequence import SamplingParams
    from .common import latent, moe, wkv, config

    cfg = config([latent(16, 128, 128, 768, 512, 128 ** -0.5, moe(4096, 8, 2, 2, 1)),
                  wkv(32, 64, moe(4096, 8, 2, 2, 1))], vocab=2000, width=2048, mult=0.5, cap=30.0)
    from replisense_rfq_amd.models.config import numalorn_from_json
    from replisense_rfq_amd.models.numalorn import NumalornLM
    from replisense_rfq_amd.models.weights import init_numalorn_weights
    from replisense_rfq_amd.engine.engine import LLMEngine
    from replisense_rfq_amd.utils.config import EngineConfig

    mcfg = numalorn_from_json(cfg, name="test-numalorn-wide")
    outs = []
    for graphs in (True, False):
        w = init_numalorn_weights(mcfg, "cuda:0", torch.bfloat16, 0, keep_full=False)
        model = NumalornLM(mcfg, "cuda:0", weights=w)
        eng = LLMEngine(EngineConfig(model="x", device="cuda:0", max_num_seqs=4, max_kv_blocks=64,
                                     max_batched_tokens=2048, max_model_len=512, use_graphs=graphs,
                                     graph_buckets=(4,), grammar=False, prefix_cache=False,
                                     warm_prefix=False, tune_gemm=False, jump_forward=False), model=model)
        prompts = [tokens(n, cfg["vocab"], 200 + n) for n in (300, 70, 200)]
        seqs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, grammar=False))
        outs.append([s.output_ids for s in seqs])
        assert bool(eng.runner.graphs) == graphs
        del eng, model, w
        torch.cuda.empty_cache()
    same = sum(a == b for x, y in zip(*outs) for a, b in zip(x, y))
    assert same >= 20, outs            # 24 tokens; a rounding tie may move a late one
