"""The kernel that draws seeded weights on the GPU against the host's function: the float64
standard normals bit for bit (which a fused multiply-add anywhere in the kernel would break), the
float32 and bfloat16 values, and a model drawn on the device against the same model written to a
folder and loaded."""
import numpy as np
import pytest

from conftest import random_prompt

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed,tensor,n", [(0, 0, 1 << 21), (2 ** 63 + 12345, 291, 1000003), (7, 2, 5), (1, 1, 4)])
def test_device_normals_are_the_hosts_bits(seed, tensor, n):
    import torch
    from sonicboom_amd import ops
    from sonicboom_amd.weights import random_stream as rs
    want = rs.standard_normals(seed, tensor, n)
    got = ops.random_normal((n,), seed, tensor, dtype=torch.float64).cpu().numpy()
    assert np.array_equal(got.view(np.uint64), want.view(np.uint64)), \
        f"{(got.view(np.uint64) != want.view(np.uint64)).sum()} of {n} float64 normals differ"
    for mean, std in ((0.0, 0.02), (1.0, 0.02)):
        f32 = ops.random_normal((n,), seed, tensor, mean, std, torch.float32).cpu().numpy()
        assert np.array_equal(f32.view(np.uint32), (want * std + mean).astype(np.float32).view(np.uint32))
        bf = ops.random_normal((n,), seed, tensor, mean, std, torch.bfloat16)
        assert torch.equal(bf.cpu(), torch.from_numpy((want * std + mean).astype(np.float32)).to(torch.bfloat16))
    # a piece that starts in the middle: elements count from `first`
    if n > 4096:
        piece = ops.random_normal((1000,), seed, tensor, dtype=torch.float64, first=4096).cpu().numpy()
        assert np.array_equal(piece, want[4096:5096])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_folder_and_the_device_give_the_same_model(tmp_path, tiny_configs, dtype):
    """write_random_model + from_folder and from_random of the same (configuration, seed, dtype)
    are one model: the same logits to the bit."""
    import torch
    from sonicboom_amd.engine import DecoderModel, Engine, StepEntry
    from sonicboom_amd.weights import write_random_model
    for name in ("A", "B"):
        cfg = tiny_configs[name]
        folder = str(tmp_path / f"{name}_{dtype}")
        write_random_model(folder, dict(cfg), seed=77, dtype=dtype, device=None)      # the host draws
        tokens = random_prompt(np.random.default_rng(1), cfg["vocab_size"], 40)
        logits = []
        for model in (DecoderModel.from_folder(folder, dtype), DecoderModel.from_random(dict(cfg), 77, dtype)):
            eng = Engine(model, 128)
            s = eng.alloc_slot()
            logits.append(eng.step([StepEntry(s, tokens, range(len(tokens)))]).cpu())
        assert torch.equal(logits[0], logits[1])
