"""Pins the oracle's whole-model forward (lo_llama_forward).

Independent evidence: a config-only (random-init, nothing downloaded) Hugging
Face LlamaForCausalLM / Qwen3ForCausalLM in fp64 loaded with the same weights
-- the textbook model the reference's LlamaModel reduces to -- plus the
cross-path identity "prefill then decode == one long prefill".
"""
import numpy as np
import pytest
import torch

from lumen_amd import synth
from oracle import lumen_oracle as lo
from tests import golden_util

transformers = pytest.importorskip("transformers")

TINY = dict(vocab_size=97, hidden_size=64, intermediate_size=176, num_hidden_layers=3, num_attention_heads=8,
            num_key_value_heads=2, rms_norm_eps=1e-5, max_seq_len=48, rope_theta=10000.0)
TINY_QWEN = dict(vocab_size=131, hidden_size=48, intermediate_size=80, num_hidden_layers=2, num_attention_heads=4,
                 num_key_value_heads=2, rms_norm_eps=1e-6, max_seq_len=40, rope_theta=1.0e6, head_dim=32,
                 qk_norm=True, tie_embeddings=True)


def hf_model(cfg, params):
    common = dict(vocab_size=cfg["vocab_size"], hidden_size=cfg["hidden_size"],
                  intermediate_size=cfg["intermediate_size"], num_hidden_layers=cfg["num_hidden_layers"],
                  num_attention_heads=cfg["num_attention_heads"], num_key_value_heads=cfg["num_key_value_heads"],
                  rms_norm_eps=cfg["rms_norm_eps"], max_position_embeddings=cfg["max_seq_len"],
                  rope_theta=cfg["rope_theta"], hidden_act="silu", attention_bias=False,
                  tie_word_embeddings=bool(cfg.get("tie_embeddings")), attn_implementation="eager")
    if cfg.get("qk_norm"):
        conf = transformers.Qwen3Config(head_dim=cfg["head_dim"], **common)
        model = transformers.Qwen3ForCausalLM(conf)
    else:
        conf = transformers.LlamaConfig(mlp_bias=False, **common)
        model = transformers.LlamaForCausalLM(conf)
    sd = {k: torch.from_numpy(v) for k, v in params.items()}
    if cfg.get("tie_embeddings"):
        sd["lm_head.weight"] = sd["model.embed_tokens.weight"]
    missing, unexpected = model.load_state_dict(sd, strict=False)
    assert not [m for m in missing if "rotary" not in m] and not unexpected, (missing, unexpected)
    return model.double().eval()


@pytest.mark.parametrize("name", golden_util.CASES)
def test_forward_matches_committed_golden_logits(name):
    """The same comparison against the committed fp64 vectors (no transformers needed at test time)."""
    cfg, params, ids, ref = golden_util.load_case(name)
    n, n_prompt = len(ids), 13
    m = lo.Llama(cfg, params)
    rc, logits = m.forward(ids[:n_prompt])
    assert rc == lo.LO_OK
    scale = np.abs(ref).max()
    assert np.abs(logits - ref[:n_prompt]).max() <= 2e-5 * scale
    for t in range(n_prompt, n):
        rc, lg = m.forward(ids[t:t + 1])
        assert rc == lo.LO_OK
        assert np.abs(lg[0] - ref[t]).max() <= 2e-5 * scale
        assert lo.argmax(lg[0]) == int(ref[t].argmax())


@pytest.mark.parametrize("cfg", [TINY, TINY_QWEN], ids=["llama", "qwen3"])
def test_forward_matches_hf_fp64(cfg):
    params = synth.make_params(cfg, seed=3, std=0.1, gains_one=False)
    ids = synth.make_tokens(20, cfg["vocab_size"], seed=3)
    hf = hf_model(cfg, params)
    with torch.no_grad():
        ref = hf(torch.from_numpy(ids.astype(np.int64))[None]).logits[0].numpy()
    m = lo.Llama(cfg, params)
    rc, logits = m.forward(ids[:13])                       # prefill, all-rows logits (llama.rs:205)
    assert rc == lo.LO_OK and m.kv_len == 13
    scale = np.abs(ref).max()
    assert np.abs(logits - ref[:13]).max() <= 2e-5 * scale
    for t in range(13, 20):                                # decode one token at a time (main.rs:367)
        rc, lg = m.forward(ids[t:t + 1])
        assert rc == lo.LO_OK and lg.shape == (1, cfg["vocab_size"])
        assert np.abs(lg[0] - ref[t]).max() <= 2e-5 * scale
        assert lo.argmax(lg[0]) == int(ref[t].argmax())
    assert m.kv_len == 20


def test_prefill_then_decode_equals_one_long_prefill_and_reset():
    params = synth.make_params(TINY, seed=5, std=0.1, gains_one=False)
    ids = synth.make_tokens(30, TINY["vocab_size"], seed=5)
    m = lo.Llama(TINY, params)
    _, full = m.forward(ids)
    m.reset()                                              # reset_kv_caches: len = 0 (llama.rs:172-176)
    assert m.kv_len == 0
    _, a = m.forward(ids[:9])
    _, b = m.forward(ids[9:17])                            # incremental prefill into a live cache (main.rs:333-335)
    rows = [a, b]
    for t in range(17, 30):
        rows.append(m.forward(ids[t:t + 1])[1])
    again = np.concatenate(rows, 0)
    assert np.abs(again - full).max() <= 1e-5 * np.abs(full).max()


def test_overflow_and_oob_status():
    params = synth.make_params(TINY, seed=7)
    m = lo.Llama(TINY, params)
    ids = synth.make_tokens(TINY["max_seq_len"], TINY["vocab_size"], seed=7)
    assert m.forward(ids)[0] == lo.LO_OK
    assert m.forward(ids[:1])[0] == lo.LO_ERR_KV_OVERFLOW  # self_attention.rs:144-149
    m.reset()
    assert m.forward(np.array([TINY["vocab_size"]]))[0] == lo.LO_ERR_EMBED_OOB  # embedding.rs:55


def test_a_cache_filled_from_outside_continues_bit_exactly():
    """lo_llama_set_kv: a second model whose caches are filled with the first one's rows (and nothing of its own
    prompt pass) decodes the same bits; rows beyond the given length are not taken; bad arguments are refused."""
    params = synth.make_params(TINY, seed=9, std=0.1, gains_one=False)
    a, b = lo.Llama(TINY, params), lo.Llama(TINY, params)
    ids = synth.make_tokens(30, TINY["vocab_size"], seed=9)
    a.forward(ids[:21])
    for layer in range(TINY["num_hidden_layers"]):
        k, v = a.cache_k(layer).copy(), a.cache_v(layer).copy()
        k[:, :, 21:], v[:, :, 21:] = 7.0, 7.0   # must not be copied
        assert b.set_kv(layer, k, v, 21) == lo.LO_OK
        assert np.array_equal(b.cache_k(layer), a.cache_k(layer)) and np.array_equal(b.cache_v(layer), a.cache_v(layer))
    assert b.kv_len == 21
    for t in range(21, 30):
        _, la = a.forward(ids[t:t + 1])
        _, lb = b.forward(ids[t:t + 1])
        assert np.array_equal(la, lb)
    k = a.cache_k(0)
    assert b.set_kv(TINY["num_hidden_layers"], k, k, 1) == lo.LO_ERR_CACHE_COUNT
    assert b.set_kv(0, k, k, TINY["max_seq_len"] + 1) == lo.LO_ERR_KV_OVERFLOW
