"""Deterministic synthetic weights and token ids for the benchmark configurations.

Every tensor gets its own PCG64 stream keyed by (seed, crc32(name)), so tensors
can be generated in any order (or lazily, one at a time) and always hold the
same bytes.  Weights are N(0, 0.02) f32, RMSNorm gains are 1.0; prompts are
uniform ids in [0, vocab).  Parameter names are the HF names the reference
exposes from LlamaModel::named_parameters (src/models/llama.rs:218-279).
"""
import zlib

import numpy as np

# --- model shapes named by the benchmark configurations ----------------------
TINYLLAMA_1B = dict(vocab_size=32000, hidden_size=2048, intermediate_size=5632, num_hidden_layers=22,
                    num_attention_heads=32, num_key_value_heads=4, rms_norm_eps=1e-5, max_seq_len=2048,
                    rope_theta=10000.0)  # src/models/llama.rs:23-37, src/main.rs:171-181
TINYLLAMA_1B_LONG = dict(TINYLLAMA_1B, max_seq_len=4096)
QWEN3_0P6B = dict(vocab_size=151936, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28,
                  num_attention_heads=16, num_key_value_heads=8, rms_norm_eps=1e-6, max_seq_len=1024,
                  rope_theta=1.0e6, head_dim=128, qk_norm=True, tie_embeddings=True)
LLAMA2_7B = dict(vocab_size=32000, hidden_size=4096, intermediate_size=11008, num_hidden_layers=32,
                 num_attention_heads=32, num_key_value_heads=32, rms_norm_eps=1e-5, max_seq_len=1024,
                 rope_theta=10000.0, weight_dtype="bf16")


def head_dim(cfg):
    return cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]


def param_shapes(cfg):
    """Ordered {hf_name: shape}; weights are [out, in] (src/layers/basic/linear.rs:8)."""
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    D = head_dim(cfg)
    qd, kvd = cfg["num_attention_heads"] * D, cfg["num_key_value_heads"] * D
    shapes = {"model.embed_tokens.weight": (V, H)}
    for i in range(cfg["num_hidden_layers"]):
        p = "model.layers.%d." % i
        shapes[p + "self_attn.q_proj.weight"] = (qd, H)
        shapes[p + "self_attn.k_proj.weight"] = (kvd, H)
        shapes[p + "self_attn.v_proj.weight"] = (kvd, H)
        shapes[p + "self_attn.o_proj.weight"] = (H, qd)
        if cfg.get("qk_norm"):
            shapes[p + "self_attn.q_norm.weight"] = (D,)
            shapes[p + "self_attn.k_norm.weight"] = (D,)
        shapes[p + "mlp.gate_proj.weight"] = (I, H)
        shapes[p + "mlp.up_proj.weight"] = (I, H)
        shapes[p + "mlp.down_proj.weight"] = (H, I)
        shapes[p + "input_layernorm.weight"] = (H,)
        shapes[p + "post_attention_layernorm.weight"] = (H,)
    shapes["model.norm.weight"] = (H,)
    if not cfg.get("tie_embeddings"):
        shapes["lm_head.weight"] = (V, H)
    return shapes


def _rng(seed, name):
    return np.random.Generator(np.random.PCG64(np.random.SeedSequence([int(seed), zlib.crc32(name.encode())])))


def is_norm_gain(name):
    return name.endswith("norm.weight") or name.endswith("layernorm.weight")


def make_param(name, shape, seed=0, std=0.02, gains_one=True):
    """One f32 tensor.  With gains_one=False the norm gains are 1 + N(0, 0.1), which
    makes a missing or misplaced gain visible in parity tests."""
    n = int(np.prod(shape))
    if is_norm_gain(name):
        if gains_one:
            return np.ones(shape, np.float32)
        return (1.0 + 0.1 * _rng(seed, name).standard_normal(n, dtype=np.float32)).reshape(shape)
    w = _rng(seed, name).standard_normal(n, dtype=np.float32)
    w *= np.float32(std)
    return w.reshape(shape)


def iter_params(cfg, seed=0, std=0.02, gains_one=True):
    for name, shape in param_shapes(cfg).items():
        yield name, make_param(name, shape, seed, std, gains_one)


def iter_params_threaded(cfg, seed=0, std=0.02, gains_one=True, workers=8, transform=None):
    """iter_params with the tensors generated (and passed through `transform(name, array)`, e.g. a bf16 rounding) by a
    pool of threads a few tensors ahead of the consumer; same bytes, same order (every tensor has its own stream)."""
    from collections import deque
    from concurrent.futures import ThreadPoolExecutor

    def job(name, shape):
        a = make_param(name, shape, seed, std, gains_one)
        return name, (transform(name, a) if transform else a)

    todo = iter(param_shapes(cfg).items())
    with ThreadPoolExecutor(max(1, workers)) as pool:
        ahead = deque()
        for name, shape in todo:
            ahead.append(pool.submit(job, name, shape))
            if len(ahead) >= 2 * workers:
                yield ahead.popleft().result()
        while ahead:
            yield ahead.popleft().result()


def make_params(cfg, seed=0, std=0.02, gains_one=True):
    return dict(iter_params(cfg, seed, std, gains_one))


def make_tokens(n, vocab, seed=0, stream="prompt"):
    return _rng(seed, stream).integers(0, vocab, size=n, dtype=np.int64).astype(np.int32)


def bf16_round(x):
    """f32 -> bf16 bits, round to nearest even (numpy, for test inputs)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    return r.astype(np.uint16)


def bf16_widen(bits):
    """bf16 bits -> f32, exact (the reference's load-time upcast, src/loader.rs:58)."""
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
