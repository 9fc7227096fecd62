"""GPU parity: whole-model forward (prefill, teacher-forced decode, greedy generation) against the
CPU oracle on the same seeded weights and token ids.

Tolerance (stated by the benchmark): per-step logits max|d|/max|ref| <= 1e-4 for f32 weights,
<= 2e-2 for bf16-stored weights (the oracle runs on the same bf16 values widened to f32); greedy
picks identical unless the oracle's top-2 logits are closer than the tolerance (an argmax tie).
"""
import numpy as np
import pytest

from lumen_amd import _lib, synth
from lumen_amd.autograd import no_grad
from lumen_amd.models import LayeredLlamaModel, LlamaModel
from oracle import lumen_oracle as lo
from tests import golden_util
from tests.gpu_util import max_rel

pytestmark = pytest.mark.gpu

TINY = dict(vocab_size=300, hidden_size=128, intermediate_size=352, num_hidden_layers=3, num_attention_heads=8,
            num_key_value_heads=2, rms_norm_eps=1e-5, max_seq_len=96, rope_theta=10000.0)
TINY_MHA = dict(TINY, num_key_value_heads=8, hidden_size=256, num_attention_heads=8)
TINY_QWEN = dict(vocab_size=411, hidden_size=96, intermediate_size=160, num_hidden_layers=2, num_attention_heads=4,
                 num_key_value_heads=2, rms_norm_eps=1e-6, max_seq_len=80, rope_theta=1.0e6, head_dim=64,
                 qk_norm=True, tie_embeddings=True)
SMALL = dict(vocab_size=2000, hidden_size=512, intermediate_size=1408, num_hidden_layers=4, num_attention_heads=8,
             num_key_value_heads=2, rms_norm_eps=1e-5, max_seq_len=256, rope_theta=10000.0)


def build(cfg, seed, std=0.1, gains_one=False, bf16=False):
    params = synth.make_params(cfg, seed=seed, std=std, gains_one=gains_one)
    gcfg = dict(cfg)
    if bf16:
        gcfg["weight_dtype"] = "bf16"
        bits = {n: synth.bf16_round(a) for n, a in params.items() if a.ndim == 2}
        params = {n: (synth.bf16_widen(bits[n]) if n in bits else a) for n, a in params.items()}
    gpu = LlamaModel(gcfg)
    for n, a in params.items():
        gpu.set_param(n, bits[n] if bf16 and n in bits and n != "model.embed_tokens.weight" else a)
    return gpu, lo.Llama(cfg, params), params


def check_argmax(got_logits, ref_logits, tol):
    ref_pick = lo.argmax(ref_logits)
    got_pick = int(np.argmax(got_logits))
    if got_pick != ref_pick:  # only a near-tie may differ
        top2 = np.sort(ref_logits)[-2:]
        assert top2[1] - top2[0] <= 2 * tol * np.abs(ref_logits).max(), (got_pick, ref_pick)


@pytest.mark.parametrize("cfg,tol,bf16", [(TINY, 1e-4, False), (TINY_MHA, 1e-4, False), (TINY_QWEN, 1e-4, False),
                                          (SMALL, 1e-4, False), (TINY, 2e-2, True), (TINY_QWEN, 2e-2, True)],
                         ids=["gqa", "mha", "qwen3", "small", "gqa-bf16", "qwen3-bf16"])
def test_prefill_then_teacher_forced_decode(cfg, tol, bf16):
    gpu, ora, _ = build(cfg, seed=11, bf16=bf16)
    n_prompt, n_dec = 19, 24
    ids = synth.make_tokens(n_prompt + n_dec, cfg["vocab_size"], seed=11)
    got = gpu.forward(ids[:n_prompt], all_rows=True)
    rc, ref = ora.forward(ids[:n_prompt])
    assert rc == lo.LO_OK and got.shape == ref.shape
    assert max_rel(got, ref) <= tol
    assert gpu.kv_len == ora.kv_len == n_prompt
    for t in range(n_prompt, n_prompt + n_dec):
        g = gpu.forward(ids[t:t + 1], all_rows=False)
        rc, r = ora.forward(ids[t:t + 1])
        assert rc == lo.LO_OK
        assert max_rel(g, r[0]) <= tol, (t, max_rel(g, r[0]))
        check_argmax(g, r[0], tol)
    assert gpu.kv_len == ora.kv_len == n_prompt + n_dec
    if not bf16:
        for layer in range(cfg["num_hidden_layers"]):
            k, v = gpu.cache(layer)
            n = n_prompt + n_dec
            assert max_rel(k[:, :, :n], ora.cache_k(layer)[:, :, :n]) <= tol
            assert max_rel(v[:, :, :n], ora.cache_v(layer)[:, :, :n]) <= tol


@pytest.mark.parametrize("name", golden_util.CASES)
def test_against_committed_golden_logits(name):
    """Prefill then decode against the committed fp64 logits of an independent implementation of the model
    (tests/golden): same 1e-4 bound as against the oracle."""
    cfg, params, ids, ref = golden_util.load_case(name)
    n, n_prompt = len(ids), 13
    gpu = LlamaModel(cfg)
    for pname, a in params.items():
        gpu.set_param(pname, a)
    got = gpu.forward(ids[:n_prompt], all_rows=True)
    assert max_rel(got, ref[:n_prompt]) <= 1e-4
    for t in range(n_prompt, n):
        g = gpu.forward(ids[t:t + 1], all_rows=False)
        assert max_rel(g, ref[t]) <= 1e-4, (t, max_rel(g, ref[t]))
        check_argmax(g, ref[t].astype(np.float32), 1e-4)


def test_last_row_only_prefill_equals_all_rows_and_incremental_prefill():
    gpu, ora, _ = build(TINY, seed=12)
    ids = synth.make_tokens(30, TINY["vocab_size"], seed=12)
    full = gpu.forward(ids, all_rows=True)
    gpu.reset_kv_caches()
    assert gpu.kv_len == 0
    last = gpu.forward(ids[:9], all_rows=False)
    assert max_rel(last, full[8]) <= 1e-5
    rest = gpu.forward(ids[9:], all_rows=True)  # prefill into a live cache (main.rs:333-335)
    assert max_rel(rest, full[9:]) <= 1e-5
    rc, ref = ora.forward(ids)
    assert max_rel(full, ref) <= 1e-4


@pytest.mark.parametrize("cfg,tol,bf16", [(TINY, 1e-4, False), (TINY_QWEN, 1e-4, False), (SMALL, 1e-4, False),
                                          (TINY, 2e-2, True)], ids=["gqa", "qwen3", "small", "gqa-bf16"])
@pytest.mark.parametrize("n", [2, 3, 4])
def test_prompts_of_two_to_four_tokens(cfg, tol, bf16, n):
    """Prompt passes of two rows take the weight-streaming product on the vector ALU (whole weight rows per wavefront,
    the rows of the prompt multiplied side by side), of three and four rows the one on the f32 matrix instruction, with
    store / residual / SwiGLU epilogues, instead of the matrix-core tiles: same branch of the reference (S > 1,
    matmul.rs:70-92), checked into an empty and into a live cache."""
    gpu, ora, _ = build(cfg, seed=30 + n, bf16=bf16)
    ids = synth.make_tokens(3 * n + 1, cfg["vocab_size"], seed=30 + n)
    got = gpu.forward(ids[:n], all_rows=True)
    rc, ref = ora.forward(ids[:n])
    assert rc == lo.LO_OK and max_rel(got, ref) <= tol
    got = gpu.forward(ids[n:2 * n], all_rows=True)          # into a live cache (main.rs:333-335)
    rc, ref = ora.forward(ids[n:2 * n])
    assert max_rel(got, ref) <= tol
    last = gpu.forward(ids[2 * n:3 * n], all_rows=False)    # what a chat turn keeps: the last row
    rc, ref = ora.forward(ids[2 * n:3 * n])
    assert max_rel(last, ref[-1]) <= tol
    one = gpu.forward(ids[3 * n:], all_rows=False)           # and a decode step on top of it
    rc, ref = ora.forward(ids[3 * n:])
    assert max_rel(one, ref[-1]) <= tol and gpu.kv_len == 3 * n + 1


@pytest.mark.parametrize("cfg", [dict(TINY, max_seq_len=128), dict(TINY_QWEN, max_seq_len=128), SMALL,
                                 dict(SMALL, hidden_size=1024, intermediate_size=2816, num_hidden_layers=2)],
                         ids=["gqa", "qwen3", "small", "wide"])
@pytest.mark.parametrize("n,bf16", [(5, False), (16, False), (17, False), (32, False), (7, True), (32, True)])
def test_prompts_of_five_to_32_tokens(cfg, n, bf16):
    """Prompt passes of three to 32 rows (16 with bf16-stored weights) take the weight-streaming matrix-core product (16 rows of a
    weight per wavefront, f32 matrix instructions, K ranges added inside the workgroup and in a second pass; store /
    residual + next norm / SwiGLU epilogues, q|k|v partials handed to the RoPE pass): same branch of the reference
    (S > 1, matmul.rs:70-92), into an empty and into a live cache, followed by a decode step.  bf16-stored weights
    are widened on their way into the operand registers (loader.rs:58 widens them at load time)."""
    tol = 2e-2 if bf16 else 1e-4
    gpu, ora, _ = build(cfg, seed=70 + n, bf16=bf16)
    ids = synth.make_tokens(3 * n + 1, cfg["vocab_size"], seed=70 + n)
    got = gpu.forward(ids[:n], all_rows=True)
    rc, ref = ora.forward(ids[:n])
    assert rc == lo.LO_OK and max_rel(got, ref) <= tol
    got = gpu.forward(ids[n:2 * n], all_rows=True)          # into a live cache (main.rs:333-335)
    rc, ref = ora.forward(ids[n:2 * n])
    assert max_rel(got, ref) <= tol
    last = gpu.forward(ids[2 * n:3 * n], all_rows=False)    # what a chat turn keeps: the last row
    rc, ref = ora.forward(ids[2 * n:3 * n])
    assert max_rel(last, ref[-1]) <= tol
    one = gpu.forward(ids[3 * n:], all_rows=False)           # and a decode step on top of it
    rc, ref = ora.forward(ids[3 * n:])
    assert max_rel(one, ref[-1]) <= tol and gpu.kv_len == 3 * n + 1


def test_greedy_generation_on_device_matches_oracle_loop():
    gpu, ora, _ = build(SMALL, seed=13)
    prompt = synth.make_tokens(12, SMALL["vocab_size"], seed=13)
    n = 40
    g_last = gpu.forward(prompt, all_rows=False)
    rc, r = ora.forward(prompt)
    first = lo.argmax(r[-1])
    assert int(np.argmax(g_last)) == first
    ids, logits = gpu.decode_greedy(first, n, want_logits=True)
    assert gpu.kv_len == 12 + n
    tok = first
    for t in range(n):
        rc, r = ora.forward(np.array([tok]))
        assert max_rel(logits[t], r[0]) <= 1e-4, t
        nxt = lo.argmax(r[0])
        if ids[t] != nxt:
            check_argmax(logits[t], r[0], 1e-4)
            pytest.skip("argmax near-tie at step %d: sequences legitimately diverge" % t)
        tok = nxt
    # the same picks again without logits, after a reset, in one call
    gpu.reset_kv_caches()
    gpu.forward(prompt, all_rows=False)
    assert np.array_equal(gpu.decode_greedy(first, n), ids)


@pytest.mark.parametrize("fused_ops", [True, False], ids=["fused-operators", "leaf-operators"])
def test_layered_operator_path_matches_fused_path_and_oracle(fused_ops):
    """LlamaModel::forward composed operator by operator: one call per reference leaf, or -- single tokens -- the
    fused operators (five launches per layer); both against the checker and the model-level path."""
    params = synth.make_params(TINY, seed=14, std=0.1, gains_one=False)
    layered = LayeredLlamaModel(TINY, params, fused=fused_ops)
    ora = lo.Llama(TINY, params)
    fused = LlamaModel(TINY)
    fused.load_params(params)
    ids = synth.make_tokens(20, TINY["vocab_size"], seed=14)
    caches = layered.init_kv_caches(1)
    with pytest.raises(NotImplementedError):  # outside no_grad the reference takes its train path
        layered.forward(ids[:15], caches)
    with no_grad():  # main.rs:255
        _layered_checks(layered, fused, ora, ids, caches)


@pytest.mark.parametrize("cfg_extra", [dict(), dict(intermediate_size=1024),
                                       dict(hidden_size=128, intermediate_size=352, max_seq_len=200)],
                         ids=["chain-3-launches", "chain+mlp-chain-2-launches", "no-chain-5-launches"])
def test_layer_level_operator_matches_the_oracle_across_a_trip_boundary(cfg_extra):
    """LlamaDecoderLayer::forward_infer for one token as ONE operator call per layer
    (lumen_decoder_layer_decode_f32): the model-level step's launches behind a layer-granular interface.  Prompt
    through the leaf operators, then single tokens through the layer operator, across 256 cached rows (a second trip
    of rows), against the checker and against the model-level path."""
    cfg = dict(CHAIN, max_seq_len=300)
    cfg.update(cfg_extra)
    params = synth.make_params(cfg, seed=61, std=0.1, gains_one=False)
    layered = LayeredLlamaModel(cfg, params, layer_op=True)
    ora = lo.Llama(cfg, params)
    fused = LlamaModel(cfg)
    fused.load_params(params)
    n_prompt = 250 if cfg["max_seq_len"] >= 300 else 20
    ids = synth.make_tokens(n_prompt + 12, cfg["vocab_size"], seed=61)
    caches = layered.init_kv_caches(1)
    with no_grad():
        a = layered.forward(ids[:n_prompt], caches).data()[0]
        _, r = ora.forward(ids[:n_prompt])
        assert max_rel(a, r) <= 1e-4
        fused.forward(ids[:n_prompt], all_rows=False)
        for t in range(n_prompt, n_prompt + 12):
            a = layered.forward(ids[t:t + 1], caches).data()[0, 0]
            _, r = ora.forward(ids[t:t + 1])
            assert max_rel(a, r[0]) <= 1e-4, t
            assert max_rel(fused.forward(ids[t:t + 1], all_rows=False), a) <= 2e-5, t
    assert caches[0].len == caches[-1].len == n_prompt + 12
    layered.ctx.synchronize()  # (would report a hand-over wait that ran out)


def _layered_checks(layered, fused, ora, ids, caches):
    a = layered.forward(ids[:15], caches).data()[0]
    rc, r = ora.forward(ids[:15])
    assert max_rel(a, r) <= 1e-4
    assert max_rel(fused.forward(ids[:15]), r) <= 1e-4
    for t in range(15, 20):
        a = layered.forward(ids[t:t + 1], caches).data()[0, 0]
        rc, r = ora.forward(ids[t:t + 1])
        assert max_rel(a, r[0]) <= 1e-4
        assert max_rel(fused.forward(ids[t:t + 1], all_rows=False), r[0]) <= 1e-4
    assert caches[0].len == 20
    with pytest.raises(_lib.LumenError) as e:
        layered.forward(ids[:1], caches[:-1])  # llama.rs:182-188
    assert e.value.status == _lib.ERR_CACHE_COUNT


def test_status_codes_for_overflow_oob_and_bad_params():
    gpu, ora, params = build(TINY, seed=15)
    ids = synth.make_tokens(TINY["max_seq_len"], TINY["vocab_size"], seed=15)
    gpu.forward(ids[:-1], all_rows=False)
    gpu.forward(ids[-1:], all_rows=False)
    assert gpu.kv_len == TINY["max_seq_len"]
    for call in (lambda: gpu.forward(ids[:1]), lambda: gpu.decode_greedy(1, 1)):
        with pytest.raises(_lib.LumenError) as e:
            call()
        assert e.value.status == _lib.ERR_KV_OVERFLOW
    gpu.reset_kv_caches()
    with pytest.raises(_lib.LumenError) as e:
        gpu.forward(np.array([TINY["vocab_size"]]))
    assert e.value.status == _lib.ERR_EMBED_OOB and gpu.kv_len == 0
    with pytest.raises(_lib.LumenError) as e:
        gpu.set_param("model.layers.0.mlp.up_proj.weight", np.zeros((3, 3), np.float32))
    assert e.value.status == _lib.ERR_SHAPE
    with pytest.raises(_lib.LumenError) as e:
        gpu.set_param("model.layers.99.mlp.up_proj.weight", np.zeros((3, 3), np.float32))
    assert e.value.status == _lib.ERR_INVALID
    with pytest.raises(_lib.LumenError) as e:
        gpu.forward(ids[:2], caches=[0])
    assert e.value.status == _lib.ERR_CACHE_COUNT


GQA64 = dict(vocab_size=1500, hidden_size=512, intermediate_size=1408, num_hidden_layers=3, num_attention_heads=8,
             num_key_value_heads=1, rms_norm_eps=1e-5, max_seq_len=512, rope_theta=10000.0)  # head_dim 64, n_rep 8
MHA128 = dict(vocab_size=700, hidden_size=256, intermediate_size=704, num_hidden_layers=2, num_attention_heads=2,
              num_key_value_heads=2, rms_norm_eps=1e-5, max_seq_len=300, rope_theta=10000.0)  # head_dim 128, n_rep 1


# The library holds no persistent decode kernel (the mode constant is kept so that callers get a clear refusal).
MODES = ("graph", "eager")


def test_persistent_mode_is_refused():
    gpu, _, _ = build(GQA64, seed=20)
    assert gpu.decode_mode == "graph"
    with pytest.raises(_lib.LumenError) as e:
        gpu.set_decode_mode("persistent")
    assert e.value.status == _lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("cfg,bf16,n_prompt", [(GQA64, False, 140), (MHA128, False, 37), (TINY_QWEN, False, 9),
                                               (GQA64, True, 33)], ids=["gqa64", "mha128", "qwen3", "gqa64-bf16"])
def test_decode_modes_agree_with_each_other_and_the_oracle(cfg, bf16, n_prompt):
    """HIP-graph replay and eager launches are two ways to issue the same step."""
    tol = 2e-2 if bf16 else 1e-4
    gpu, ora, _ = build(cfg, seed=21, bf16=bf16)
    ids = synth.make_tokens(n_prompt + 6, cfg["vocab_size"], seed=21)
    rc, ref_prompt = ora.forward(ids[:n_prompt])
    refs = [ora.forward(ids[t:t + 1])[1][0] for t in range(n_prompt, n_prompt + 6)]
    first = lo.argmax(refs[-1])
    tok, greedy_ref = first, []
    for _ in range(5):
        r = ora.forward(np.array([tok]))[1][0]
        greedy_ref.append(r)
        tok = lo.argmax(r)
    results = {}
    for mode in MODES:
        gpu.reset_kv_caches()
        gpu.set_decode_mode(mode)
        gpu.forward(ids[:n_prompt], all_rows=False)
        rows = [gpu.forward(ids[t:t + 1], all_rows=False) for t in range(n_prompt, n_prompt + 6)]
        picks, logits = gpu.decode_greedy(first, 5, want_logits=True)
        assert gpu.kv_len == n_prompt + 11
        for g, r in zip(rows, refs):
            assert max_rel(g, r) <= tol, mode
        for t in range(5):
            assert max_rel(logits[t], greedy_ref[t]) <= tol, (mode, t)
            check_argmax(logits[t], greedy_ref[t], tol)
        results[mode] = (np.stack(rows), picks, logits)
    assert np.array_equal(results["graph"][0], results["eager"][0])  # same kernels, same order of operations
    assert np.array_equal(results["graph"][1], results["eager"][1])


@pytest.mark.parametrize("cfg_extra,n_prompt", [
    (dict(num_attention_heads=8, num_key_value_heads=1, max_seq_len=640), 505),             # head_dim 64, n_rep 8: 512
    (dict(num_attention_heads=8, num_key_value_heads=2, max_seq_len=1100), 506),            # n_rep 4, 16 slices offered
    (dict(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, max_seq_len=330, intermediate_size=704), 250),  # head_dim 128: 256
    (dict(num_attention_heads=8, num_key_value_heads=2, max_seq_len=600, qk_norm=True, head_dim=64), 507),  # norm in the kernel
    (dict(hidden_size=384, num_attention_heads=6, num_key_value_heads=2, max_seq_len=600, intermediate_size=1056), 508),  # groups of three heads
    (dict(hidden_size=128, num_attention_heads=2, num_key_value_heads=1, max_seq_len=4096, intermediate_size=352), 3900),  # 16 slices, all in use
    (dict(num_attention_heads=8, num_key_value_heads=2, max_seq_len=4096), 505),  # 16 slices offered, 1 to 3 in use: merged by o_proj
    (dict(num_attention_heads=8, num_key_value_heads=2, max_seq_len=4096), 3),    # the same model from an almost empty cache
], ids=["d64-nrep8", "d64-nrep4", "d128-nrep2", "d64-qknorm", "d64-nrep3", "d64-long-4096", "d64-4096-cross", "d64-4096-start"])
def test_decode_across_the_short_to_split_attention_boundary(cfg_extra, n_prompt):
    """Decode attention changes form where the cache passes 512 rows (256 for head_dim 128): steps on both sides of
    the boundary, and the step that crosses it, agree with the checker."""
    cfg = dict(vocab_size=900, hidden_size=512, intermediate_size=1408, num_hidden_layers=2, rms_norm_eps=1e-5,
               rope_theta=10000.0)
    cfg.update(cfg_extra)
    gpu, ora, _ = build(cfg, seed=33)
    ids = synth.make_tokens(n_prompt + 14, cfg["vocab_size"], seed=33)
    got = gpu.forward(ids[:n_prompt], all_rows=False)
    rc, ref = ora.forward(ids[:n_prompt])
    assert rc == lo.LO_OK and max_rel(got, ref[-1]) <= 1e-4
    for t in range(n_prompt, n_prompt + 14):
        g = gpu.forward(ids[t:t + 1], all_rows=False)
        _, r = ora.forward(ids[t:t + 1])
        assert max_rel(g, r[0]) <= 1e-4, t
    assert gpu.kv_len == n_prompt + 14


def _greedy_call_checked(gpu, ora, first, n, tol):
    """ONE decode_greedy call of n steps; the checker is then fed the GPU's own picks, so every step's
    logits are compared on identical inputs whatever a near-tie does to the sequence."""
    picks, logits = gpu.decode_greedy(first, n, want_logits=True)
    tok = first
    for t in range(n):
        _, r = ora.forward(np.array([tok]))
        assert max_rel(logits[t], r[0]) <= tol, (t, max_rel(logits[t], r[0]))
        check_argmax(logits[t], r[0], tol)
        tok = int(picks[t])
    return picks, logits


@pytest.mark.parametrize("cfg_extra,n_prompt,same_bits", [
    (dict(num_attention_heads=8, num_key_value_heads=2, max_seq_len=4096), 492, False),  # slices merged by o_proj when eager
    (dict(num_attention_heads=8, num_key_value_heads=1, max_seq_len=4096), 490, False),  # n_rep 8: remapped head index
    (dict(num_attention_heads=8, num_key_value_heads=2, max_seq_len=1100, qk_norm=True, head_dim=64), 494, True),  # norm + rotation in the kernel
    (dict(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, max_seq_len=700, intermediate_size=704), 236, False),  # head_dim 128: 256 rows
    (dict(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, max_seq_len=700, intermediate_size=704, qk_norm=True, head_dim=128), 236, True),
], ids=["d64-nrep4-defer", "d64-nrep8-defer", "d64-qknorm", "d128", "d128-qknorm"])
def test_one_greedy_call_crosses_the_attention_boundary(cfg_extra, n_prompt, same_bits):
    """A single decode_greedy call that starts on the short side of the attention boundary (512 cached rows, 256
    for head_dim 128) and ends on the long side: the step's graph is recorded anew at the step that crosses it (the
    recorded launches carry the form to run), inside the one call.  Every step of such a call is held to the
    checker, and to the eager launches of the same steps (where the eager steps leave the merge of the slices to
    o_proj the two differ in summation order, elsewhere they are bit-equal)."""
    cfg = dict(vocab_size=900, hidden_size=512, intermediate_size=1408, num_hidden_layers=2, rms_norm_eps=1e-5,
               rope_theta=10000.0)
    cfg.update(cfg_extra)
    gpu, ora, _ = build(cfg, seed=41)
    ids = synth.make_tokens(n_prompt, cfg["vocab_size"], seed=41)
    n = 40
    results = {}
    for mode in MODES:
        gpu.reset_kv_caches()
        ora.reset()
        gpu.set_decode_mode(mode)
        got = gpu.forward(ids, all_rows=False)
        _, ref = ora.forward(ids)
        assert max_rel(got, ref[-1]) <= 1e-4
        results[mode] = _greedy_call_checked(gpu, ora, lo.argmax(ref[-1]), n, 1e-4)
        assert gpu.kv_len == n_prompt + n
    (pg, lg), (pe, le) = results["graph"], results["eager"]
    if same_bits:
        assert np.array_equal(lg, le) and np.array_equal(pg, pe)
    elif np.array_equal(pg, pe):
        assert max_rel(lg, le) <= 1e-5


CHAIN = dict(vocab_size=1200, hidden_size=512, intermediate_size=1408, num_hidden_layers=3, num_attention_heads=8,
             num_key_value_heads=2, rms_norm_eps=1e-5, max_seq_len=700, rope_theta=10000.0)  # head_dim 64, n_rep 4


@pytest.mark.parametrize("cfg_extra,bf16", [(dict(), False), (dict(num_key_value_heads=8), False),
                                            (dict(hidden_size=1024, num_attention_heads=8, num_key_value_heads=4,
                                                  intermediate_size=1024), False),
                                            (dict(hidden_size=1024, num_attention_heads=16, num_key_value_heads=2,
                                                  intermediate_size=1024), True),
                                            (dict(hidden_size=2048, num_attention_heads=16, num_key_value_heads=4,
                                                  intermediate_size=512, num_hidden_layers=2), False),
                                            (dict(hidden_size=2048, num_attention_heads=32, num_key_value_heads=4,
                                                  intermediate_size=512, num_hidden_layers=2), True),
                                            (dict(hidden_size=512, num_attention_heads=8, num_key_value_heads=4, head_dim=128,
                                                  qk_norm=True, tie_embeddings=True, rope_theta=1.0e6, rms_norm_eps=1e-6), False),
                                            (dict(hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
                                                  qk_norm=True, intermediate_size=1024, num_hidden_layers=2), True),
                                            (dict(hidden_size=512, num_attention_heads=8, num_key_value_heads=8, head_dim=128,
                                                  intermediate_size=1024, num_hidden_layers=2), False),
                                            (dict(intermediate_size=3072), False),
                                            (dict(hidden_size=1024, num_attention_heads=16, num_key_value_heads=4,
                                                  intermediate_size=2048, num_hidden_layers=2), True)],
                         ids=["d64-nrep4", "d64-mha", "d128-nrep2", "d64-nrep8-bf16", "d128-nrep4-h2048",
                              "d64-nrep8-h2048-bf16", "qwen-d128-nrep2-wide", "qwen-d128-nrep4-bf16", "d128-mha-wide", "mlp-chain-3072",
                              "mlp-chain-2048-bf16"])
def test_chained_launches_equal_the_separate_launches_they_replace(cfg_extra, bf16):
    """Short caches: decode attention and o_proj run as one launch whose attention workgroups hand their output to
    the o_proj workgroups through tagged words (form 1), with the RMSNorm + q|k|v + RoPE product in front handing q
    and the new row to the attention workgroups the same way (form 2).  Same steps with separate launches (form 0): the attention arithmetic is the same code, so
    logits agree to rounding of the sums; every form is held to the checker; the cache crosses a trip boundary
    (256 rows, 128 for head_dim 128) on the way.  q/k-norm models (head_dim 128) take form 2 with un-rotated
    projections handed over -- norm, rotation and cache write happen in the attention workgroups; o_proj rows may be
    twice as long as the q|k|v rows (n_head * head_dim = 2 * hidden).  Where the intermediate size allows (a
    multiple of 1024 values of f32 / 2048 of bf16 weights up to 16 loads per lane) forms 1 and 2 also run gate|up and
    down as one launch (act handed over as tagged words); form 0 takes that apart as well."""
    cfg = dict(CHAIN)
    cfg.update(cfg_extra)
    tol = 2e-2 if bf16 else 1e-4
    gpu, ora, _ = build(cfg, seed=51, bf16=bf16)
    n_prompt, n = 120, 150
    ids = synth.make_tokens(n_prompt, cfg["vocab_size"], seed=51)
    out = {}
    for enable in (2, 1, 0):
        if enable == 1 and cfg.get("qk_norm"):  # form 1 wants a rotated q from an earlier launch: not with q/k norm
            with pytest.raises(_lib.LumenError) as e:
                gpu.set_handover(enable=1)
            assert e.value.status == _lib.ERR_UNSUPPORTED
            continue
        gpu.set_handover(enable=enable)
        gpu.reset_kv_caches()
        ora.reset()
        last = gpu.forward(ids, all_rows=False)
        _, ref = ora.forward(ids)
        assert max_rel(last, ref[-1]) <= tol
        out[enable] = _greedy_call_checked(gpu, ora, lo.argmax(ref[-1]), n, tol)
        assert gpu.kv_len == n_prompt + n
    p0, l0 = out[0]
    for enable in (1, 2):
        if enable in out and np.array_equal(out[enable][0], p0):
            assert max_rel(out[enable][1], l0) <= (2e-6 if enable == 1 else 2e-5)


def test_attention_oproj_launch_gives_up_a_wait_that_cannot_end_in_time_and_says_so():
    """Failure handling of the hand-over inside the chained launches, forced from the host: with a poll limit of
    zero and no pauses the waiting workgroups look once, before their producers can have finished, give up and flag
    it; every wavefront exits, the call returns LUMEN_ERR_HIP, and after the defaults are back the model works."""
    gpu, ora, _ = build(CHAIN, seed=52)
    ids = synth.make_tokens(40, CHAIN["vocab_size"], seed=52)
    for enable in (1, 2):
        gpu.reset_kv_caches()
        last = gpu.forward(ids, all_rows=False)
        gpu.set_handover(enable=enable, spin_limit=0, pre_sleep=0, poll_delay=0, poll_gap=0)
        with pytest.raises(_lib.LumenError) as e:
            gpu.decode_greedy(int(np.argmax(last)), 3)
        assert e.value.status == _lib.ERR_HIP and "gave up waiting" in str(e.value)
    gpu.set_handover(enable=1, spin_limit=1 << 22, pre_sleep=11, poll_delay=17, poll_gap=1)
    gpu.set_handover(enable=2, pre_sleep=55, poll_delay=15, poll_gap=1)
    gpu.reset_kv_caches()
    last = gpu.forward(ids, all_rows=False)
    _, ref = ora.forward(ids)
    assert max_rel(last, ref[-1]) <= 1e-4
    _greedy_call_checked(gpu, ora, lo.argmax(ref[-1]), 12, 1e-4)
    for enable in (1, 2):  # a q/k-norm model with head_dim 64: no form covers it
        with pytest.raises(_lib.LumenError) as e:
            build(TINY_QWEN, seed=1)[0].set_handover(enable=enable)
        assert e.value.status == _lib.ERR_UNSUPPORTED
    # n_head * head_dim = 2 * hidden with head_dim 64
    wide = build(dict(CHAIN, num_attention_heads=16, num_key_value_heads=4, head_dim=64, num_hidden_layers=1), seed=2)[0]
    wide.set_handover(enable=1)
    with pytest.raises(_lib.LumenError) as e:  # o_proj rows twice as long as the q|k|v rows: head_dim 128 only
        wide.set_handover(enable=2)
    assert e.value.status == _lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("qk_norm", [False, True], ids=["merge-in-oproj", "merge-in-kernel"])
def test_sliced_attention_decode_is_bit_reproducible(qk_norm):
    """The same 64 greedy steps at ~4000 cached rows (16 slices per head, partial states handed from
    workgroup to workgroup through memory) give the same bits every time, whether the slices are merged by
    the attention kernel's last workgroup (q/k-norm model) or by the o_proj product."""
    cfg = dict(vocab_size=900, hidden_size=256, intermediate_size=704, num_hidden_layers=2, rms_norm_eps=1e-5,
               rope_theta=10000.0, num_attention_heads=4, num_key_value_heads=2, max_seq_len=4096)
    if qk_norm:
        cfg.update(qk_norm=True, head_dim=64)
    gpu, ora, _ = build(cfg, seed=43)
    ids = synth.make_tokens(3960, cfg["vocab_size"], seed=43)
    first = None
    for rep in range(20):
        gpu.reset_kv_caches()
        last = gpu.forward(ids, all_rows=False)
        picks, logits = gpu.decode_greedy(int(np.argmax(last)), 64, want_logits=True)
        if first is None:
            first = (last, picks, logits)
            _, ref = ora.forward(ids)
            assert max_rel(last, ref[-1]) <= 1e-4
            tok = int(np.argmax(last))
            for t in range(64):
                _, r = ora.forward(np.array([tok]))
                assert max_rel(logits[t], r[0]) <= 1e-4, t
                tok = int(picks[t])
        else:
            assert np.array_equal(last, first[0]), rep
            assert np.array_equal(picks, first[1]), rep
            assert np.array_equal(logits, first[2]), rep


@pytest.mark.slow
def test_tinyllama_1b_shape_prefill_128_decode_teacher_forced():
    """The headline configuration at full size: 22 layers, hidden 2048, 32/4 heads, vocab 32000,
    128 random prompt ids then teacher-forced decode; per-step logits within 1e-4."""
    cfg = synth.TINYLLAMA_1B
    gpu = LlamaModel(cfg)
    params = {}
    for name, a in synth.iter_params(cfg, seed=0):
        gpu.set_param(name, a)
        params[name] = a
    ora = lo.Llama(cfg, params)
    ids = synth.make_tokens(128 + 16, cfg["vocab_size"], seed=0)
    got = gpu.forward(ids[:128], all_rows=False)
    rc, ref = ora.forward(ids[:128])
    assert rc == lo.LO_OK
    assert max_rel(got, ref[-1]) <= 1e-4
    worst = 0.0
    for t in range(128, 144):
        g = gpu.forward(ids[t:t + 1], all_rows=False)
        rc, r = ora.forward(ids[t:t + 1])
        worst = max(worst, max_rel(g, r[0]))
        check_argmax(g, r[0], 1e-4)
    assert worst <= 1e-4, worst
    # on-device greedy loop reproduces itself and advances the cache
    a = gpu.decode_greedy(int(ids[0]), 8)
    assert gpu.kv_len == 144 + 8 and a.shape == (8,)
    # a follow-up turn of 12 and one of 20 tokens into the live cache: at this width the gate|up product of the
    # weight-streaming prompt kernel runs unsplit, with the SwiGLU epilogue inside (one and two row tiles)
    gpu.reset_kv_caches()
    ora.reset()
    turn = synth.make_tokens(12 + 20, cfg["vocab_size"], seed=3)
    for lo_i, hi_i in ((0, 12), (12, 32)):
        got = gpu.forward(turn[lo_i:hi_i], all_rows=True)
        rc, ref = ora.forward(turn[lo_i:hi_i])
        assert rc == lo.LO_OK and max_rel(got, ref) <= 1e-4


def _stream_build(cfg, seed, bf16=False):
    """Full-width shapes: tensors are generated a few at a time (by a pool of threads) and shared by the GPU model
    and the oracle; bf16-stored weights go to the GPU as bits and to the oracle as the same values widened."""
    gcfg = dict(cfg, weight_dtype="bf16") if bf16 else dict(cfg)
    gpu = LlamaModel(gcfg)
    params = {}

    def to_bf16(name, a):
        if a.ndim != 2:
            return a
        bits = synth.bf16_round(a)
        return bits, synth.bf16_widen(bits)

    for name, a in synth.iter_params_threaded(cfg, seed=seed, workers=12, transform=to_bf16 if bf16 else None):
        if isinstance(a, tuple):
            bits, a = a
            gpu.set_param(name, a if name == "model.embed_tokens.weight" and not cfg.get("tie_embeddings") else bits)
        else:
            gpu.set_param(name, a)
        params[name] = a
    ocfg = {k: v for k, v in cfg.items() if k != "weight_dtype"}
    return gpu, lo.Llama(ocfg, params)


def _seed_checker_with_gpu_cache(gpu, ora, length):
    """The checker goes on from the rows the GPU's prompt pass left: its own prompt pass at these sizes would take
    minutes.  (What the rows hold is then checked through what the checker computes FROM them.)"""
    for layer in range(gpu.config.num_hidden_layers):
        k, v = gpu.cache(layer)
        assert ora.set_kv(layer, k, v, length) == lo.LO_OK
    assert ora.kv_len == length


def _prefill_decode_check(gpu, ora, vocab, n_prompt, n_dec, tol, seed):
    ids = synth.make_tokens(n_prompt + n_dec, vocab, seed=seed)
    got = gpu.forward(ids[:n_prompt], all_rows=False)
    rc, ref = ora.forward(ids[:n_prompt])
    assert rc == lo.LO_OK
    assert max_rel(got, ref[-1]) <= tol, max_rel(got, ref[-1])
    worst = 0.0
    for t in range(n_prompt, n_prompt + n_dec):
        g = gpu.forward(ids[t:t + 1], all_rows=False)
        rc, r = ora.forward(ids[t:t + 1])
        worst = max(worst, max_rel(g, r[0]))
        check_argmax(g, r[0], tol)
    assert worst <= tol, worst
    assert gpu.kv_len == ora.kv_len == n_prompt + n_dec


@pytest.mark.slow
def test_long_context_tinyllama_shape_3968_prompt_decode_to_the_last_row():
    """Config 3 at full width and full context on 3 of the 22 layers (every kernel shape and the 16-slice
    attention merge are the real ones): prompt 3968, 12 teacher-forced steps, then ONE greedy call of 116
    steps that fills the 4096-row cache to its last row; the step after that is refused like the
    reference's assert (self_attention.rs:144-149)."""
    cfg = dict(synth.TINYLLAMA_1B_LONG, num_hidden_layers=3)
    gpu, ora = _stream_build(cfg, seed=3)
    _prefill_decode_check(gpu, ora, cfg["vocab_size"], 3968, 12, 1e-4, seed=3)
    _greedy_call_checked(gpu, ora, 17, 116, 1e-4)
    assert gpu.kv_len == ora.kv_len == cfg["max_seq_len"] == 4096
    k, _ = gpu.cache(2)
    assert max_rel(k[:, :, 4090:], ora.cache_k(2)[:, :, 4090:]) <= 1e-4 and np.abs(k[:, :, 4095]).max() > 0
    for call in (lambda: gpu.forward(np.array([1]), all_rows=False), lambda: gpu.decode_greedy(1, 1)):
        with pytest.raises(_lib.LumenError) as e:
            call()
        assert e.value.status == _lib.ERR_KV_OVERFLOW
    assert gpu.kv_len == 4096


@pytest.mark.slow
def test_qwen3_0p6b_shape_full_depth_prefill_256_decode():
    """Config 4 at full size: 28 layers, head_dim 128 decoupled from hidden 1024, per-head q/k RMSNorm, tied
    151936-row embedding, rope_theta 1e6; prompt 256 (the last prompt row crosses nothing: head_dim 128 changes
    form at 256 rows, so the first decode step is the first sliced one), 8 teacher-forced steps and one greedy
    call of 8.  No reference model exists for this shape (oracle-extrapolated)."""
    cfg = dict(synth.QWEN3_0P6B)
    gpu, ora = _stream_build(cfg, seed=4)
    _prefill_decode_check(gpu, ora, cfg["vocab_size"], 256, 8, 1e-4, seed=4)
    _greedy_call_checked(gpu, ora, 23, 8, 1e-4)


@pytest.mark.slow
def test_llama2_7b_shape_bf16_weights_prefill_512_decode():
    """Config 5 shape (hidden 4096, 32-head MHA, head_dim 128, intermediate 11008, bf16-stored weights,
    f32 accumulate and f32 KV cache) on 2 of the 32 layers; tolerance 2e-2 against the oracle run on the
    same bf16 values widened to f32."""
    cfg = dict(synth.LLAMA2_7B, num_hidden_layers=2)
    cfg.pop("weight_dtype")
    gpu, ora = _stream_build(cfg, seed=5, bf16=True)
    _prefill_decode_check(gpu, ora, cfg["vocab_size"], 512, 8, 2e-2, seed=5)


@pytest.mark.slow
@pytest.mark.parametrize("bf16,tol", [(False, 1e-4), (True, 2e-2)])
def test_wide_model_prompt_of_4000_rows_on_the_large_gemm_tiles(bf16, tol):
    """A prompt of 4000 rows against projections 3328 and 3840 rows wide: q|k|v and o_proj then run on the
    256x256 GEMM tiles without a K split, i.e. with the plain store and the residual add in the tile
    epilogue (TinyLlama's own widths split K there and add in a second pass), with f32 and with bf16-stored
    weights.  One layer, 52 query heads on 4 KV heads."""
    cfg = dict(vocab_size=256, hidden_size=3328, intermediate_size=256, num_hidden_layers=1,
               num_attention_heads=52, num_key_value_heads=4, rms_norm_eps=1e-5, max_seq_len=4096,
               rope_theta=10000.0)
    gpu, ora = _stream_build(cfg, seed=6, bf16=bf16)
    _prefill_decode_check(gpu, ora, cfg["vocab_size"], 4000, 2, tol, seed=6)



@pytest.mark.slow
def test_long_context_tinyllama_shape_at_full_depth_to_the_last_row():
    """Config 3 as configured: all 22 layers, 3968-token prompt, decode to row 4095 of the 4096-row cache.
    The checker does not repeat the prompt pass (minutes on the CPU): its caches are filled with the first 3967
    rows the GPU's prompt pass wrote, and from there everything is its own arithmetic --
    * its decode step for prompt token 3967 against the LAST ROW of the GPU's prompt pass (matrix-core kernels),
    * 16 teacher-forced decode steps and ONE greedy call of 112 steps up to the last row (GEMV / attention kernels),
      every step's logits within 1e-4,
    * the cache rows both sides appended in the last layer."""
    cfg = dict(synth.TINYLLAMA_1B_LONG)
    gpu, ora = _stream_build(cfg, seed=0)
    n_prompt, n_forced = 3968, 16
    ids = synth.make_tokens(n_prompt + n_forced, cfg["vocab_size"], seed=0)
    last = gpu.forward(ids[:n_prompt], all_rows=False)
    _seed_checker_with_gpu_cache(gpu, ora, n_prompt - 1)
    _, r = ora.forward(ids[n_prompt - 1:n_prompt])
    assert max_rel(last, r[0]) <= 1e-4, max_rel(last, r[0])
    check_argmax(last, r[0], 1e-4)
    worst = 0.0
    for t in range(n_prompt, n_prompt + n_forced):
        g = gpu.forward(ids[t:t + 1], all_rows=False)
        _, r = ora.forward(ids[t:t + 1])
        worst = max(worst, max_rel(g, r[0]))
        check_argmax(g, r[0], 1e-4)
    assert worst <= 1e-4, worst
    _greedy_call_checked(gpu, ora, lo.argmax(r[0]), cfg["max_seq_len"] - n_prompt - n_forced, 1e-4)
    assert gpu.kv_len == ora.kv_len == cfg["max_seq_len"]
    k, v = gpu.cache(cfg["num_hidden_layers"] - 1)
    lo_k, lo_v = ora.cache_k(cfg["num_hidden_layers"] - 1), ora.cache_v(cfg["num_hidden_layers"] - 1)
    assert max_rel(k[:, :, n_prompt - 1:], lo_k[:, :, n_prompt - 1:]) <= 1e-4
    assert max_rel(v[:, :, n_prompt - 1:], lo_v[:, :, n_prompt - 1:]) <= 1e-4
    with pytest.raises(_lib.LumenError) as e:
        gpu.decode_greedy(1, 1)
    assert e.value.status == _lib.ERR_KV_OVERFLOW


@pytest.mark.slow
def test_llama2_7b_shape_bf16_weights_at_full_depth():
    """Config 5 as configured: all 32 layers (13 GB of bf16 weights on the GPU, the same values widened to f32 --
    26 GB of host memory -- for the checker), 512-token prompt, decode across 512 -> 576 cached rows.
    * checker (caches filled with the GPU's first 511 rows, then its own arithmetic): its decode step for prompt
      token 511 against the last row of the GPU's prompt pass, and 12 steps of ONE greedy call, within 2e-2;
    * the two GPU paths against each other at every one of 64 steps: logits of decode step t (GEMV / attention
      kernels) against the last row of a prompt pass over the same t + 1 tokens (matrix-core kernels);
    * graph replay against eager launches of the same 64 steps: the same bits."""
    cfg = dict(synth.LLAMA2_7B)
    cfg.pop("weight_dtype")
    gpu, ora = _stream_build(cfg, seed=5, bf16=True)
    n_prompt, n = 512, 64
    ids = synth.make_tokens(n_prompt, cfg["vocab_size"], seed=5)
    last = gpu.forward(ids, all_rows=False)
    _seed_checker_with_gpu_cache(gpu, ora, n_prompt - 1)
    _, r = ora.forward(ids[n_prompt - 1:])
    assert max_rel(last, r[0]) <= 2e-2, max_rel(last, r[0])
    check_argmax(last, r[0], 2e-2)
    first = int(np.argmax(last))
    picks, logits = gpu.decode_greedy(first, n, want_logits=True)
    assert gpu.kv_len == n_prompt + n
    tok, worst = first, 0.0
    for t in range(12):
        _, r = ora.forward(np.array([tok]))
        worst = max(worst, max_rel(logits[t], r[0]))
        check_argmax(logits[t], r[0], 2e-2)
        tok = int(picks[t])
    assert worst <= 2e-2, worst
    # eager launches of the same steps
    gpu.set_decode_mode("eager")
    gpu.reset_kv_caches()
    assert np.array_equal(gpu.forward(ids, all_rows=False), last)
    picks_e, logits_e = gpu.decode_greedy(first, n, want_logits=True)
    gpu.set_decode_mode("graph")
    assert np.array_equal(picks_e, picks) and np.array_equal(logits_e, logits)
    # decode step t against a prompt pass over the same t + 1 tokens
    seq = np.concatenate([ids, [first], picks]).astype(np.int32)
    cross = 0.0
    for t in range(n):
        gpu.reset_kv_caches()
        row = gpu.forward(seq[:n_prompt + t + 1], all_rows=False)
        cross = max(cross, max_rel(logits[t], row))
    assert cross <= 1e-3, cross
