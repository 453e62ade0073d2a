"""Full-size model configurations of the baseline against fixtures written by the CPU oracle
(tests/golden/model_greedy.json, made by tests/golden/make_model_goldens.py; the oracle needs
minutes per configuration, so it does not run inside the suite).

Gates: greedy token ids identical over the first 64 generated tokens (32 after the 2048-token prompt of "c4", the
7B-width prefill workload, whose GEMMs and attention run the large-tile kernels).  Logits: at this size the
CPU path's own fp32 arithmetic is 3.4e-3 (max-abs) away from a float64 evaluation of the same
model (fixture "fp64_step0", tests/golden/make_fp64_probe.py), so two different fp32 summation
orders cannot agree to 1e-3; asserted instead: GPU-vs-float64 error no larger than the CPU
path's (x1.25), and GPU-vs-oracle <= FULL_SIZE_LOGIT_ATOL.  (The 1e-3 gate is asserted on the
small models in test_gpu_model.py.)  The DeepSeek fixture scales the MLA projections by 0.25: with the
reference's initialiser at this width the attention softmax is a hard arg-max (scores with a standard
deviation near 150) and two correct fp32 implementations diverge by O(1) within a few layers (see
tests/golden/make_model_goldens.py).  "g2" is the GPT path (LayerNorm, GELU, learned positions) at the size
of GPT-2 small.  Also size-independent properties at full size: graph
replay == eager, decode row == prefill row (KV-cache causality)."""
import json
import os

import numpy as np
import pytest

from deepj_amd import (DeepSeekConfig, DeepSeekModel, GPTConfig, GPTModel, JavaRandom, LlamaConfig, LlamaModel,
                       TextGenerator)

pytestmark = pytest.mark.gpu

PATH = os.path.join(os.path.dirname(__file__), "golden", "model_greedy.json")
GOLD = json.load(open(PATH)) if os.path.exists(PATH) else {}
FULL_SIZE_LOGIT_ATOL = 5e-3


MLA_PROJECTIONS = ("wdq", "wuq", "wdkv", "wuk", "wuv")


def seeded_deepseek_with_scaled_mla(cfg, seed, scale, latent_cache=False):
    """new DeepSeekModel(cfg, seed) (DeepSeekModel.java:31-47: embedding from Random(seed), the block
    stack from its own Random(seed), the LM head from Random(seed+1); Tensor.random = N(0,1)*0.1) with the
    five MLA projection matrices multiplied by `scale`, loaded through setWeight."""
    model = DeepSeekModel(cfg, None, latent_cache=latent_cache)
    emb_r, stack_r, head_r = JavaRandom(seed), JavaRandom(seed), JavaRandom(seed + 1)
    d = cfg.dModel
    model.setWeight("emb", emb_r.tensor(cfg.vocabSize, d))
    shapes = dict(wdq=(d, cfg.qRank), wuq=(cfg.qRank, d), wdkv=(d, cfg.kvRank), wuk=(cfg.kvRank, d),
                  wuv=(cfg.kvRank, d), wo=(d, d), wg=(d, cfg.dFF), wu=(d, cfg.dFF), wd=(cfg.dFF, d))
    for l in range(cfg.nLayers):
        model.setWeight(f"L{l}.g1", np.ones((1, d), np.float32))
        model.setWeight(f"L{l}.g2", np.ones((1, d), np.float32))
        for w, (r, c) in shapes.items():
            t = stack_r.tensor(r, c)
            model.setWeight(f"L{l}.{w}", t * np.float32(scale) if w in MLA_PROJECTIONS else t)
        for b, n in (("bg", cfg.dFF), ("bu", cfg.dFF), ("bd", d)):
            model.setWeight(f"L{l}.{b}", np.zeros((1, n), np.float32))
    model.setWeight("gf", np.ones((1, d), np.float32))
    model.setWeight("wlm", head_r.tensor(d, cfg.vocabSize))
    model.setWeight("blm", np.zeros((1, cfg.vocabSize), np.float32))
    model.finalize()
    return model


def build(name):
    c = GOLD[name]["config"]
    m = c["model"]
    if "q_rank" in m:
        cfg = DeepSeekConfig(m["vocab"], m["max_seq"], m["d"], m["heads"], m["layers"], m["dff"], m["q_rank"], m["kv_rank"])
        if "mla_weight_scale" in c:
            return seeded_deepseek_with_scaled_mla(cfg, c["seed"], c["mla_weight_scale"]), c
        return DeepSeekModel(cfg, c["seed"]), c
    if m.get("gpt"):
        cfg = GPTConfig(m["vocab"], m["max_seq"], m["d"], m["heads"], m["layers"], m["dff"], initScale=m["init_scale"])
        return GPTModel(cfg, c["seed"]), c
    cfg = LlamaConfig(m["vocab"], m["max_seq"], m["d"], m["heads"], m["layers"], m["dff"])
    return LlamaModel(cfg, c["seed"]), c


def logit_gate(name):
    """Max-abs gate for GPU-vs-oracle logits of a full-size fixture: the baseline's 1e-3 wherever the oracle itself is
    well inside it relative to float64 (fixture "fp64_step0": 2e-4 for "c5" and "g2"), FULL_SIZE_LOGIT_ATOL where the
    oracle's own fp32 arithmetic is already further than 1e-3 from exact ("c3": 3.4e-3, "c4")."""
    f = GOLD[name].get("fp64_step0")
    if f and f["oracle_max_abs_err_all_cols"] <= 2.5e-4:
        return 1e-3
    return FULL_SIZE_LOGIT_ATOL


@pytest.mark.parametrize("name", ["c3", "c4", "c5", "g2"])
def test_full_size_greedy_tokens_and_logits_match_oracle_fixture(name):
    if name not in GOLD:
        pytest.skip(f"no fixture for {name} (run tests/golden/make_model_goldens.py {name})")
    g = GOLD[name]
    assert "fp64_step0" in g, "every full-size fixture carries the float64 probe that justifies its logit gate"
    FULL_SIZE_LOGIT_ATOL = logit_gate(name)      # noqa: N806 - shadows the module default for this configuration
    model, c = build(name)
    try:
        prompt = JavaRandom(c["prompt_seed"]).ints(c["prompt_len"], c["model"]["vocab"])
        assert [int(x) for x in prompt[:8]] == g["prompt_head"]
        n_new = c["new_tokens"]
        # step 0: logits of the last prompt row
        model.reset()
        model.prefill(prompt, choose_next=False)
        l0 = model.lastLogits()
        probe = g["logit_probe_cols"]
        assert np.max(np.abs(l0[probe] - np.array(g["logit_probe_step0"]))) <= FULL_SIZE_LOGIT_ATOL
        assert abs(float(l0.max()) - g["top_logit"][0]) <= FULL_SIZE_LOGIT_ATOL
        if "fp64_step0" in g:
            f = g["fp64_step0"]
            exact, cpu = np.array(f["fp64"]), np.array(f["oracle_fp32"])
            gpu_err = float(np.max(np.abs(l0[f["cols"]] - exact)))
            cpu_err = float(np.max(np.abs(cpu - exact)))
            print(f"\n[{name}] max-abs error vs float64 on {len(exact)} logits: GPU {gpu_err:.2e}, CPU oracle {cpu_err:.2e}; "
                  f"GPU vs oracle {float(np.max(np.abs(l0[f['cols']] - cpu))):.2e} (gate {FULL_SIZE_LOGIT_ATOL:g})")
            assert gpu_err <= 1.25 * cpu_err + 1e-4
            assert float(np.max(np.abs(l0[f["cols"]] - cpu))) <= FULL_SIZE_LOGIT_ATOL
        # greedy generation through the captured graph
        got = TextGenerator.generate(model, prompt, n_new, top_k=1, use_graph=True)
        exp = np.array(g["tokens"], dtype=np.int32)
        assert np.array_equal(got[c["prompt_len"]:], exp), f"first mismatch at token {int(np.argmax(got[c['prompt_len']:] != exp))}"
        last = model.lastLogits()
        assert np.max(np.abs(last[probe] - np.array(g["logit_probe_last"]))) <= FULL_SIZE_LOGIT_ATOL
        print(f"\n[{name}] {n_new} greedy tokens identical; oracle min top-1/top-2 gap {g['min_top2_gap']:.4f}")
        # eager execution of the same stream gives the same ids
        eager = TextGenerator.generate(model, prompt, 16, top_k=1, use_graph=False)
        assert np.array_equal(eager[c["prompt_len"]:], exp[:16])
        # decode row == prefill row at full size
        ids = np.concatenate([prompt[:40], exp[:3]])
        full = model.forward(ids)
        model.reset()
        model.prefill(ids[:40], choose_next=False)
        for t in range(40, 43):
            model.step(int(ids[t]))
            assert float(np.max(np.abs(model.lastLogits() - full[t]))) <= FULL_SIZE_LOGIT_ATOL
    finally:
        model.close()


def test_full_size_deepseek_with_the_latent_cache_matches_the_fixture():
    """The "c5" fixture again with cKV cached instead of K and V (runner kind 3): step-0 logits inside the same
    gate, the 64 greedy tokens identical."""
    g = GOLD.get("c5")
    if not g:
        pytest.skip("no c5 fixture")
    c, m = g["config"], g["config"]["model"]
    cfg = DeepSeekConfig(m["vocab"], m["max_seq"], m["d"], m["heads"], m["layers"], m["dff"], m["q_rank"], m["kv_rank"])
    model = seeded_deepseek_with_scaled_mla(cfg, c["seed"], c["mla_weight_scale"], latent_cache=True)
    try:
        prompt = JavaRandom(c["prompt_seed"]).ints(c["prompt_len"], m["vocab"])
        model.reset()
        model.prefill(prompt, choose_next=False)
        l0 = model.lastLogits()
        f = g["fp64_step0"]
        assert float(np.max(np.abs(l0[f["cols"]] - np.array(f["oracle_fp32"])))) <= logit_gate("c5")
        got = TextGenerator.generate(model, prompt, c["new_tokens"], top_k=1, use_graph=True)
        assert np.array_equal(got[c["prompt_len"]:], np.array(g["tokens"], dtype=np.int32))
    finally:
        model.close()


# ── the DeepSeek configuration exactly as stated: reference initialisation, nothing scaled ─────────────────────
#
# At this width the reference's initialiser (N(0,1) * 0.1) gives attention scores with a standard deviation near 150:
# every softmax row is a hard arg-max, a near-tie between the two best keys flips with the summation order, and one
# flip replaces a whole value row.  The fixture's float64 probe measures the consequence on the CPU side alone: the
# oracle's fp32 logits of the last prompt row are 4.8 (max-abs; 1.2 rms, logits of +-20) away from the float64 value,
# and a second fp32 evaluation in numpy's summation order is 4.3 away from the oracle.  "Token-identical to the CPU
# path" is therefore not a property any other summation order can have at this initialisation - two CPU orders do not
# have it either - and the model is checked in the ways that stay meaningful:
#   * end to end: GPU-vs-float64 distance no larger than the CPU path's own (x1.25); greedy ids identical to the
#     oracle's under teacher forcing up to the first step whose oracle top-1/top-2 gap is below the measured
#     GPU-vs-oracle distance (that step is reported); graph replay == eager (bit-identical kernels);
#   * block by block: every tested block of the 16, fed the oracle's own input to that block, agrees with the oracle
#     (prefill rows and cached decode rows) - the check that does not compound.

def seeded_deepseek_weights(cfg, seed):
    """The parameters of new DeepSeekModel(cfg, seed) by name (DeepSeekModel.java:31-47, draw order of
    DeepSeekTransformerBuilder.java:56-68), from the java.util.Random twin."""
    emb_r, stack_r, head_r = JavaRandom(seed), JavaRandom(seed), JavaRandom(seed + 1)
    d = cfg.dModel
    w = {"emb": emb_r.tensor(cfg.vocabSize, d)}
    shapes = dict(wdq=(d, cfg.qRank), wuq=(cfg.qRank, d), wdkv=(d, cfg.kvRank), wuk=(cfg.kvRank, d),
                  wuv=(cfg.kvRank, d), wo=(d, d), wg=(d, cfg.dFF), wu=(d, cfg.dFF), wd=(cfg.dFF, d))
    for l in range(cfg.nLayers):
        w[f"L{l}.g1"] = np.ones((1, d), np.float32)
        w[f"L{l}.g2"] = np.ones((1, d), np.float32)
        for name, (r, c) in shapes.items():
            w[f"L{l}.{name}"] = stack_r.tensor(r, c)
        for b, n in (("bg", cfg.dFF), ("bu", cfg.dFF), ("bd", d)):
            w[f"L{l}.{b}"] = np.zeros((1, n), np.float32)
    w["gf"] = np.ones((1, d), np.float32)
    w["wlm"] = head_r.tensor(d, cfg.vocabSize)
    w["blm"] = np.zeros((1, cfg.vocabSize), np.float32)
    return w


def test_deepseek_at_the_stated_init_end_to_end():
    name = "c5_ref_init"
    if name not in GOLD or "fp64_step0" not in GOLD[name]:
        pytest.skip("no fixture (run tests/golden/make_model_goldens.py c5_ref_init and make_fp64_probe.py c5_ref_init)")
    g, f = GOLD[name], GOLD[name]["fp64_step0"]
    model, c = build(name)
    try:
        prompt = JavaRandom(c["prompt_seed"]).ints(c["prompt_len"], c["model"]["vocab"])
        assert [int(x) for x in prompt[:8]] == g["prompt_head"]
        exp = np.array(g["tokens"], dtype=np.int32)
        # step 0 against float64 and against the oracle
        model.reset()
        model.prefill(prompt, choose_next=False)
        l0 = model.lastLogits()
        exact, cpu = np.array(f["fp64"]), np.array(f["oracle_fp32"])
        gpu_err = float(np.max(np.abs(l0[f["cols"]] - exact)))
        cpu_err = float(np.max(np.abs(cpu - exact)))
        dist = float(np.max(np.abs(l0[f["cols"]] - cpu)))
        print(f"\n[{name}] step 0, max-abs over {len(exact)} logits: GPU vs float64 {gpu_err:.3f}, oracle vs float64 "
              f"{cpu_err:.3f} (all columns {f['oracle_max_abs_err_all_cols']:.3f}; a second CPU fp32 order "
              f"{f['alt_fp32_max_abs_err_all_cols']:.3f}), GPU vs oracle {dist:.3f}")
        assert np.all(np.isfinite(l0))
        assert gpu_err <= 1.25 * max(cpu_err, f["oracle_max_abs_err_all_cols"])
        # teacher forcing: the GPU sees the oracle's tokens; its arg-max may leave the oracle's only at a step whose
        # oracle gap is below the measured distance
        first_part, agree = None, 0
        for t, (i1, l1, i2, l2) in enumerate(g["steps"]):
            if t > 0:
                model.step(int(exp[t - 1]))
            same = int(np.argmax(model.lastLogits())) == i1
            agree += same
            if not same and first_part is None:
                first_part = t
                assert l1 - l2 < dist, (f"step {t}: the GPU leaves the oracle's token although the oracle's top-1/top-2 "
                                        f"gap {l1 - l2:.3f} exceeds the GPU-vs-oracle logit distance {dist:.3f}")
        print(f"[{name}] teacher-forced arg-max equals the oracle's at {agree} of {len(exp)} steps; first parting at step "
              f"{first_part} (oracle gap there {g['steps'][first_part][1] - g['steps'][first_part][3]:.3f})"
              if first_part is not None else f"[{name}] all {len(exp)} teacher-forced steps agree")
        # the GPU's own greedy sequence: graph replay and eager launches run the same kernels on the same data
        a = TextGenerator.generate(model, prompt, 24, top_k=1, use_graph=True)
        b = TextGenerator.generate(model, prompt, 24, top_k=1, use_graph=False)
        assert np.array_equal(a, b)
        # decode row against prefill row: two GPU summation orders (matvec and GEMM kernels) of a model whose CPU
        # orders are O(1) apart; reported, and bounded by the CPU path's own distance from float64
        ids = np.concatenate([prompt[:40], exp[:3]])
        full = model.forward(ids)
        model.reset()
        model.prefill(ids[:40], choose_next=False)
        worst = 0.0
        for t in range(40, 43):
            model.step(int(ids[t]))
            worst = max(worst, float(np.max(np.abs(model.lastLogits() - full[t]))))
        print(f"[{name}] decode row vs prefill row at full depth: max-abs {worst:.3f}")
        assert worst <= 1.25 * f["oracle_max_abs_err_all_cols"]
    finally:
        model.close()


@pytest.mark.parametrize("layer", range(16))
def test_deepseek_at_the_stated_init_block_by_block(layer, stated_init):
    """Block `layer` of the 16-block model at the stated initialisation, fed the oracle's own input to that block:
    a one-block GPU model whose embedding table holds those input rows against a one-block oracle with the same
    weights.  Prefill rows (GEMM kernels) and cached decode rows (matvec kernels, KV cache)."""
    cfg, w, cpu16, ids = stated_init
    check_block(layer, cfg, w, cpu16, ids)


@pytest.mark.parametrize("layer", (0, 7, 15))
def test_deepseek_at_the_stated_init_block_by_block_at_the_config_prompt_length(layer, stated_init):
    """The same check on the configuration's own prompt, 256 ids from Random(5): the first, a middle and the last
    block.  With five times the rows there are five times the chances that two keys of a (hard arg-max) softmax row
    nearly tie, and block 0 - whose scores are the largest relative to its input - shows it: measured 6 of its 256 rows
    between 1.0e-3 and 1.64e-3 from the oracle (the same rows, to the digit, with every GEMM forced onto the bf16
    kernels: it is the summation order inside attention, not a kernel's precision), median row 9e-5; blocks 7 and
    15 stay below 3e-4.  Gate: at least 97 % of the rows within the baseline's 1e-3, the worst within 2.5e-3."""
    cfg, w, cpu16, _ = stated_init
    check_block(layer, cfg, w, cpu16, JavaRandom(5).ints(256, cfg.vocabSize), worst_row=2.5e-3, rows_within=0.97)


def check_block(layer, cfg, w, cpu16, ids, worst_row=1e-3, rows_within=1.0):
    from oracle import cpu_ref as ref
    S, d = len(ids), cfg.dModel
    x_in = cpu16.hidden(ids, layer)                                  # [S x d], what block `layer` sees on the CPU
    one = DeepSeekConfig(S, S, d, cfg.nHeads, 1, cfg.dFF, cfg.qRank, cfg.kvRank)     # vocabulary = the S input rows
    names = ("g1", "g2", "wdq", "wuq", "wdkv", "wuk", "wuv", "wo", "wg", "bg", "wu", "bu", "wd", "bd")
    head = np.ascontiguousarray(w["wlm"][:, :S])
    gpu = DeepSeekModel(one, None)
    cpu = ref.Model(vocab=S, max_seq=S, d=d, heads=cfg.nHeads, layers=1, dff=cfg.dFF, seed=1, q_rank=cfg.qRank,
                    kv_rank=cfg.kvRank, timing_only_fill=True)
    try:
        for n in names:
            gpu.setWeight(f"L0.{n}", w[f"L{layer}.{n}"])
            cpu.weight(f"L0.{n}")[...] = w[f"L{layer}.{n}"]
        for n, v in (("emb", x_in), ("gf", w["gf"]), ("wlm", head), ("blm", np.zeros((1, S), np.float32))):
            gpu.setWeight(n, v)
            cpu.weight(n)[...] = v
        gpu.finalize()
        cpu.q8_roundtrip()
        rows = np.arange(S, dtype=np.int32)
        exp = cpu.forward(rows)
        got = gpu.forward(rows)
        per_row = np.max(np.abs(got - exp), axis=1)
        err = float(np.max(per_row))
        within = float(np.mean(per_row <= 1e-3))
        scale = float(np.sqrt(np.mean(exp.astype(np.float64) ** 2)))
        gpu.reset()
        gpu.prefill(rows[:S - 4], choose_next=False)
        derr = 0.0
        for t in range(S - 4, S):
            gpu.step(int(rows[t]))
            derr = max(derr, float(np.max(np.abs(gpu.lastLogits() - exp[t]))))
        print(f"\n[c5 stated init, block {layer}, {S} rows] input rms {float(np.sqrt(np.mean(x_in.astype(np.float64) ** 2))):.2f}, "
              f"logit rms {scale:.2f}: prefill rows max-abs {err:.2e}, decode rows {derr:.2e}")
        print(f"    rows within 1e-3: {within:.3f}")
        assert err <= worst_row and within >= rows_within and derr <= 1e-3      # 1e-3: the baseline's logit tolerance
    finally:
        gpu.close()
        cpu.close()


@pytest.fixture(scope="module")
def stated_init():
    """The 16-block DeepSeek model of the baseline at its stated initialisation on the CPU oracle (weights from the
    java.util.Random twin, which tests/test_host_random.py pins bit for bit to the oracle's), and a 48-token prompt."""
    from oracle import cpu_ref as ref
    m = GOLD["c5_ref_init"]["config"]["model"] if "c5_ref_init" in GOLD else dict(
        vocab=32000, max_seq=512, d=2048, heads=16, layers=16, dff=5632, q_rank=1024, kv_rank=512)
    cfg = DeepSeekConfig(m["vocab"], m["max_seq"], m["d"], m["heads"], m["layers"], m["dff"], m["q_rank"], m["kv_rank"])
    w = seeded_deepseek_weights(cfg, 42)
    ref.set_threads(ref.default_threads())
    cpu16 = ref.Model(vocab=cfg.vocabSize, max_seq=cfg.maxSeqLen, d=cfg.dModel, heads=cfg.nHeads, layers=cfg.nLayers,
                      dff=cfg.dFF, seed=42, q_rank=cfg.qRank, kv_rank=cfg.kvRank, timing_only_fill=True)
    for n in cpu16.weight_names():
        cpu16.weight(n)[...] = w[n]
    cpu16.q8_roundtrip()
    ids = JavaRandom(5).ints(48, cfg.vocabSize)
    yield cfg, w, cpu16, ids
    cpu16.close()
    ref.set_threads(1)
