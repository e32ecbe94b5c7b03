"""A sweep of configurations of sizes that the two tiny models do not have: head sizes in steps
of 16 up to 256, groups of 1 to 17 query heads per key/value head, widths, inner sizes and
vocabularies that are no power of two and no multiple of a tile, one to three layers, tied and
untied heads, head_dim given or left to follow from the width.  Each is drawn from a seed,
written as a model folder with random weights, and run in float32 and bfloat16 against the plain
implementation: every request whole, with its tail token by token, and in a batch of unequal
prompts; no page may be left held afterwards.  Widths of 2,048 and more are held to the bfloat16
bounds of real layer sizes (rows that long round as those do), the others to the tiny models'."""
import numpy as np
import pytest

from helpers import assert_logits_close, forget_plain, plain_logits, run_batch, run_tail_one_by_one, run_whole

pytestmark = pytest.mark.gpu

HEAD_SIZES = (16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256)
GROUPS = (1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17)
LENGTHS = (3, 17, 63, 64, 65, 100, 129, 200)


def drawn_config(seed):
    """The configuration and the prompt lengths of a seed.  Seed i takes head size i and group i
    of the lists above, so that twelve seeds go through all of both; the rest is drawn."""
    rng = np.random.default_rng(1000 + seed)
    hd = HEAD_SIZES[seed % len(HEAD_SIZES)]
    group = GROUPS[(seed * 5) % len(GROUPS)]
    hkv = int(rng.choice([1, 2, 3, 5]))
    while hd * hkv * group > 4096 and hkv > 1:
        hkv -= 1
    while hd * hkv * group > 4096:
        group -= 1
    heads = hkv * group
    hidden = heads * hd                    # the architecture refuses any other width
    cfg = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "num_hidden_layers": int(rng.integers(1, 4)), "hidden_size": hidden,
        "num_attention_heads": heads, "num_key_value_heads": hkv,
        "intermediate_size": int(rng.choice([40, 100, 136, 257, 300, 520, 1000])),
        "vocab_size": int(rng.choice([97, 257, 1000, 1531, 4099])),
        "rope_theta": float(rng.choice([10000.0, 5e5, 1e6])),
        "rms_norm_eps": float(rng.choice([1e-6, 1e-5, 3e-4])),
        "max_position_embeddings": 1024, "tie_word_embeddings": bool(rng.integers(0, 2)),
        "hidden_act": "silu",
    }
    if seed % 3 == 0:
        cfg["head_dim"] = hd
    lengths = [int(n) for n in rng.choice(LENGTHS, size=3, replace=False)]
    return cfg, lengths, rng


def _name(seed):
    cfg, _, _ = drawn_config(seed)
    hd = cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    return (f"hd{hd}-q{cfg['num_attention_heads']}-kv{cfg['num_key_value_heads']}-w{cfg['hidden_size']}"
            f"-ff{cfg['intermediate_size']}-v{cfg['vocab_size']}-L{cfg['num_hidden_layers']}")


@pytest.mark.parametrize("seed", range(12), ids=_name)
def test_odd_sizes_whole_tail_and_batch(tmp_path, seed):
    from sonicboom_amd.engine import DecoderModel, Engine
    from sonicboom_amd.weights import write_random_model

    cfg, lengths, rng = drawn_config(seed)
    folder = str(tmp_path / "model")
    write_random_model(folder, dict(cfg), seed=100 + seed, dtype="bfloat16")
    requests = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lengths]
    prompt_lengths = [max(1, n // 2) for n in lengths]
    kind = "wide" if cfg["hidden_size"] >= 2048 else False
    try:
        for dtype in ("float32", "bfloat16"):
            engine = Engine(DecoderModel.from_folder(folder, dtype), 64 * 24)
            for tokens in requests:
                want = plain_logits(folder, tokens)
                assert_logits_close(run_whole(engine, tokens), want, dtype, f"{dtype} whole", kind)
                assert_logits_close(run_tail_one_by_one(engine, tokens), want, dtype, f"{dtype} tail", kind)
            got = run_batch(engine, requests, prompt_lengths)
            for tokens, p, g in zip(requests, prompt_lengths, got):
                want = plain_logits(folder, tokens)
                assert_logits_close(g, want[p - 1:] if g.shape[0] != len(tokens) else want, dtype, f"{dtype} batch",
                                    kind)
            assert engine.cache.held_pages() == 0
            del engine
    finally:
        forget_plain(folder)
