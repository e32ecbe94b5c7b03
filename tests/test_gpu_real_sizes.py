"""The engine against the plain implementation at real layer sizes: two layers of the widths,
head counts, head size and vocabulary of the benchmark configuration (width 3,584, 28 heads on 4
kv heads of 128, inner width 18,944, 152,064 tokens, separate head), loaded from a folder of
about 3 GB.  At these sizes the launchers take the choices the measurements take (the
weight-streaming products and their K cuts, the 256 x 256 tiles, the decode attention's chunks,
the head's own form), which the tiny models never reach; and random N(0, 0.02) weights give
attention scores of a few units by themselves.  One request whole and with its last 32 tokens one
by one, a batch of 8 and a batch of 64 unequal requests, in 32-bit and in bfloat16."""
import time

import numpy as np
import pytest

from conftest import random_prompt
from helpers import assert_logits_close, forget_plain, plain_logits, plain_model, run_batch, run_tail_one_by_one, run_whole

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 4096, "tie_word_embeddings": False, "use_sliding_window": False,
    "hidden_act": "silu",
}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from sonicboom_amd.weights import write_random_model
    path = str(tmp_path_factory.mktemp("real_sizes"))
    t0 = time.time()
    write_random_model(path, dict(CONFIG), seed=4242, dtype="bfloat16")
    print(f"[real sizes] folder written in {time.time() - t0:.1f} s", flush=True)
    plain_model(path, wide=True)
    yield path
    forget_plain(path)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes(folder, dtype):
    import torch
    from sonicboom_amd.engine import DecoderModel, Engine
    vocab = CONFIG["vocab_size"]
    rng = np.random.default_rng(5)
    t0 = time.time()
    model = DecoderModel.from_folder(folder, dtype)
    torch.cuda.synchronize()
    print(f"[real sizes] {dtype} model loaded in {time.time() - t0:.1f} s, "
          f"{torch.cuda.max_memory_allocated() / 2**30:.1f} GiB at most on the device", flush=True)
    eng = Engine(model, 64 * 2 * 64)
    one = random_prompt(rng, vocab, 64)
    want = plain_logits(folder, one)
    assert_logits_close(run_whole(eng, one), want, dtype, "whole", sharp="wide")
    assert_logits_close(run_tail_one_by_one(eng, one), want, dtype, "last 32 one by one", sharp="wide")
    for n_req, longest in ((8, 90), (64, 40)):
        prompts = [int(n) for n in rng.integers(1, longest, size=n_req)]
        prompts[0], prompts[-1] = 1, longest          # a one-token prompt and the longest
        decoded = [int(n) for n in rng.integers(1, 5, size=n_req)]
        reqs = [random_prompt(rng, vocab, p + d) for p, d in zip(prompts, decoded)]
        got = run_batch(eng, reqs, prompts)
        for i, (r, g) in enumerate(zip(reqs, got)):
            assert_logits_close(g, plain_logits(folder, r), dtype, f"batch of {n_req}, request {i}", sharp="wide")
        assert eng.cache.held_pages() == 0 and not eng.cache.live_slots
    # the same model drawn on the device (the folder's seed and stored type): the same bits
    from sonicboom_amd.engine import StepEntry
    drawn = Engine(DecoderModel.from_random(dict(CONFIG), 4242, dtype, stored="bfloat16"), 128)
    logits = []
    for e in (eng, drawn):
        s = e.alloc_slot()
        logits.append(e.step([StepEntry(s, one, range(len(one)))]).cpu())
        e.free_slot(s)
    assert torch.equal(logits[0], logits[1]), "the model drawn on the device is not the folder's"
    del eng, model, drawn
    torch.cuda.empty_cache()
