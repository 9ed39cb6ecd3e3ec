"""The engine at widths the tiny configurations do not reach: two layers at the Llama-3.1-8B layer
sizes with the full vocabulary, a model of 18 query heads on one key/value head, and a hidden
size of 2,304, an intermediate size of 5,120; whole, in portions, and with the last tokens one by one, against the plain
implementation, in 32-bit and in bfloat16."""
import numpy as np
import pytest

import plain_llama
from helpers import check_rounding_noise, check_steps_against, cut_portions, cut_tail_single, cut_whole, random_requests, run_steps, scaled_tol

pytestmark = pytest.mark.gpu

WIDE = {
    # two layers of the 8B shape: hidden 4096, 32 query heads on 8 of 128, intermediate 14336, vocabulary 128256
    "E": dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=4096, intermediate_size=14336,
              num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=128, vocab_size=128256,
              max_position_embeddings=1024, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=False,
              rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                original_max_position_embeddings=256), hidden_act="silu", eos_token_id=128001),
    # 18 query heads share one key/value head (more than the matrix-core attention kernels group), hidden 2304
    "K": dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=2304, intermediate_size=1184,
              num_hidden_layers=2, num_attention_heads=18, num_key_value_heads=1, head_dim=128, vocab_size=1000,
              max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True,
              hidden_act="silu", eos_token_id=999),
    # hidden 2560 (no power of two), groups of 5 on head size 64
    "M": dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=2560, intermediate_size=1760,
              num_hidden_layers=3, num_attention_heads=20, num_key_value_heads=4, head_dim=64, vocab_size=1500,
              max_position_embeddings=512, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=False,
              hidden_act="silu", eos_token_id=1499),
    # an intermediate size of 5,120: portions of 33..64 tokens take the fused gate/up kernel whose blocks
    # hold four groups of waves (E: two groups)
    "G": dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=1024, intermediate_size=5120,
              num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=4, head_dim=64, vocab_size=2000,
              max_position_embeddings=512, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True,
              hidden_act="silu", eos_token_id=1999),
}
LENGTHS = {"E": [600, 70], "K": [300, 45, 130], "M": [257, 64, 400], "G": [300, 70, 41]}


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    """name -> (model folder, requests, plain logits), made when first asked for."""
    made = {}

    def get(name):
        if name not in made:
            from rustinfer_amd.config import LlamaConfig
            from rustinfer_amd.weights import write_random_model
            d = str(tmp_path_factory.mktemp(f"wide_{name}"))
            write_random_model(LlamaConfig.from_dict(WIDE[name]), 40 + len(made), d)
            cfg, w = plain_llama.read_model(d)
            reqs = random_requests(cfg["vocab_size"], LENGTHS[name], seed=61)
            plain = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
            del w
            made[name] = (d, reqs, plain)
        return made[name]
    return get


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name", ["K", "M", "G", "E"])
def test_wide_models_match_plain_under_three_cuts(wide, name, dtype):
    from rustinfer_amd.engine import build_engine
    d, reqs, plain = wide(name)
    tol = scaled_tol(dtype, plain)
    eng = build_engine(d, dtype=dtype, page_size=16, num_pages=80, max_requests=4,
                       max_model_len=WIDE[name]["max_position_embeddings"], max_batch_tokens=1024)
    for cut, steps in (("whole", cut_whole(reqs)), ("portions", cut_portions(reqs, seed=7)),
                       ("tail_single", cut_tail_single(reqs, tail=32))):
        results = run_steps(eng, steps)
        if dtype == "float32":
            worst = check_steps_against(steps, results, plain, tol, f"{name}/{dtype}/{cut}")
            print(f"{name} {dtype} {cut}: worst |diff| {worst:.3e} of {tol:.3e}")
        else:
            # bfloat16 at these widths: errors are rounding noise that grows with width and depth
            # (0.8 % of the logits' deviation at K, 1.1 % at M); what is checked is that it is noise
            med, spread = check_rounding_noise(steps, results, plain, f"{name}/{dtype}/{cut}")
            print(f"{name} {dtype} {cut}: median row error {med:.2%} of the deviation, largest row {spread:.2f} x median")
        eng.cache.check()
        assert eng.cache.free_pages() == 80


@pytest.mark.parametrize("rows,copies", [(40, 2), (24, 2), (12, 2), (12, 1), (40, 1)])
def test_many_requests_decode_together_at_real_widths(wide, rows, copies):
    """Steps of 40 or 24 single tokens at the 8B widths: the few-row products with the activations
    in LDS (q/k/v with rotation and cache write, gate/up, o and down as partial sums); of 12: o adds
    to the residual stream itself and leaves the norm to gate/up, down (a large weight, more than
    eight rows) goes as partial sums with the norm's own kernel.  With one copy of the weights
    (no tile-ordered second one) the products of these sizes go to the GEMM library, rotation and
    norms to kernels of their own.  In bfloat16 against the plain implementation."""
    d, _, _ = wide("E")
    cfg, w = plain_llama.read_model(d)
    reqs = random_requests(cfg["vocab_size"], [14] * rows, seed=77)
    plain = {r: plain_llama.forward(cfg, w, t) for r, t in reqs.items()}
    del w
    from rustinfer_amd.engine import build_engine
    eng = build_engine(d, dtype="bfloat16", page_size=16, num_pages=80, max_requests=48,
                       max_model_len=WIDE["E"]["max_position_embeddings"], max_batch_tokens=1024,
                       tiled_weight_copy=copies == 2)
    assert (eng.model.layers[0].ffn.down.weight_tiled is not None) == (copies == 2)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:8], "want": [7]} for r, t in reqs.items()], "end": []}]
    for p in range(8, 14):
        steps.append({"step": len(steps), "entries": [{"id": r, "tokens": [t[p]], "want": [0]} for r, t in reqs.items()],
                      "end": list(reqs) if p == 13 else []})
    results = run_steps(eng, steps)
    med, spread = check_rounding_noise(steps, results, plain, f"E/bfloat16/{rows} rows/{copies} copies")
    print(f"E bfloat16 {rows} single tokens, {copies} copies: median row error {med:.2%} of the deviation, largest row {spread:.2f} x median")
    eng.cache.check()
    assert eng.cache.free_pages() == 80


LONG = {
    # one layer at the 8B layer sizes, two at the 1B ones; a vocabulary of 8,192 keeps the head small
    "8b": dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=4096, intermediate_size=14336,
               num_hidden_layers=1, num_attention_heads=32, num_key_value_heads=8, head_dim=128, vocab_size=8192,
               max_position_embeddings=8192, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=False),
    "1b": dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=2048, intermediate_size=8192,
               num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8, head_dim=64, vocab_size=8192,
               max_position_embeddings=8192, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True),
}


@pytest.mark.parametrize("name", ["8b", "1b"])
def test_long_contexts_at_real_widths_against_the_32_bit_path(tmp_path, name):
    """Contexts of 2,000 to 3,000 tokens at the benchmark's layer sizes, where the plain
    implementation would take minutes: the bfloat16 engine (graphs on, also for steps with
    portions) against the 32-bit engine on the same trace, step by step.  The trace holds whole
    prompts, portions behind hundreds and thousands of cached keys beside single tokens (keys
    divided between blocks, several blocks a (kv head, token) pair), and single tokens of 2 to 8
    requests under graphs; no kind of step may stand out from bfloat16's rounding."""
    import json
    import os
    import torch
    from rustinfer_amd.engine import StepEntry, build_engine
    d = str(tmp_path)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(LONG[name], f)
    engs = {dt: build_engine(d, dtype=dt, page_size=16, num_pages=900, max_requests=8, max_model_len=4096,
                             max_batch_tokens=4096, random_weights_seed=7) for dt in ("float32", "bfloat16")}
    engs["bfloat16"].enable_graphs(True, (1, 2, 4, 8), mixed_tokens=512)
    reqs = random_requests(LONG[name]["vocab_size"], [2300, 2100, 700, 40, 3000, 1500, 2200, 90], seed=5)
    names = list(reqs)
    pos = {r: 0 for r in reqs}
    R = lambda *idx: [names[i] for i in idx]
    plans = [[(names[0], 2048)], [(names[1], 2048), (names[0], 1)], [(names[0], 1), (names[1], 1), (names[2], 256)],
             [(names[0], 1), (names[1], 1), (names[2], 256), (names[3], 16)], [(names[4], 2900)],
             [(names[0], 1), (names[1], 1), (names[2], 100), (names[3], 1), (names[4], 1)],
             [(names[5], 1400), (names[6], 2100)], [(r, 1) for r in R(0, 1, 2, 3, 4, 5, 6)],
             [(names[7], 64)] + [(r, 1) for r in R(0, 1, 2, 3, 4, 5, 6)], [(names[7], 2), (names[0], 1), (names[4], 2)]]
    plans += [[(r, 1) for r in R(0, 1, 2, 4, 5, 6, 7)]] * 6 + [[(r, 1) for r in R(0, 4)]] * 3
    for i, plan in enumerate(plans):
        ents = [StepEntry(r, reqs[r][pos[r]:pos[r] + n], [n - 1]) for r, n in plan]
        a = engs["float32"].step(ents).float()
        b = engs["bfloat16"].step(ents).float()
        torch.cuda.synchronize()
        rel = ((a - b).abs().max() / a.abs().max()).item()
        assert rel < 0.04, (name, i, plan[:3], rel)
        for r, n in plan:
            pos[r] += n
    graphs = engs["bfloat16"]._graphs
    assert any(k[0] == "mixed" and k[-1] == 1 for k in graphs) and any(k[0] != "mixed" and k[1] >= 3072 for k in graphs)
    for e in engs.values():
        e.cache.check()
