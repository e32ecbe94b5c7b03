"""Long rows: the attention kernels at 16,384 and 32,768 keys, rotation at positions of tens of
thousands, and a prompt of 20,000 tokens through the engine, which runs it in two portions.  Random
keys move an output over 32,768 keys by less than any tolerance, so beside random data one key at
a time is made to dominate (in the first, a middle and the last chunk of the row): the output must
then be that key's value."""
import math

import numpy as np
import pytest
import torch

from conftest import random_prompt
from helpers import assert_logits_close
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16


def close(got, want, atol, rtol, what=""):
    got = got.detach().float().cpu().numpy().astype(np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want)
    assert got.shape == want.shape and (err <= atol + rtol * np.abs(want)).all(), \
        f"{what}: max |diff| {err.max():.3g} at {np.unravel_index(np.argmax(err), err.shape)}"


def paged(keys, vals, seed):
    """bfloat16 caches holding one sequence's ``keys`` and ``vals`` [n, hkv, hd] on scattered pages;
    returns (keys, values, page table [1, pages])."""
    from sonicboom_amd.cache import layout
    n, hkv, hd = keys.shape
    width = (n + 63) // 64
    table = torch.randperm(width + 7, generator=torch.Generator().manual_seed(seed))[:width].to(torch.int32)
    pad = width * 64 - n
    k = torch.cat([keys, torch.full((pad, hkv, hd), float("nan"))]).reshape(width, 64, hkv, hd).permute(0, 2, 1, 3)
    v = torch.cat([vals, torch.full((pad, hkv, hd), float("nan"))]).reshape(width, 64, hkv, hd).permute(0, 2, 3, 1)
    kc = torch.full((width + 7, hkv, 64, hd), float("nan"), dtype=BF16)
    vc = torch.full((width + 7, hkv, hd, 64), float("nan"), dtype=BF16)
    # the cache keeps the elements of a row in an order of its own: scatter to where each lies
    kpos = torch.from_numpy(layout.key_positions(hd)).expand(width, hkv, 64, hd)
    vpos = torch.from_numpy(layout.value_positions(hd)).expand(width, hkv, hd, 64)
    kc[table.long()] = torch.empty_like(k, dtype=BF16).scatter_(-1, kpos, k.to(BF16).contiguous())
    vc[table.long()] = torch.empty_like(v, dtype=BF16).scatter_(-1, vpos, v.to(BF16).contiguous())
    return kc.to(DEV), vc.to(DEV), table[None, :].contiguous()


def looking_along_zero(n, hq, hkv, hd, n_rows, seed):
    """Small random keys and queries whose coordinate 0 is large in the queries: a key whose
    coordinate 0 is raised by ``rise`` scores 56 above the rest and takes all of a row's weight."""
    g = torch.Generator().manual_seed(seed)
    scale = 1.0 / math.sqrt(hd)
    keys = (torch.randn(n, hkv, hd, generator=g) * 0.05).to(BF16).float()
    vals = torch.randn(n, hkv, hd, generator=g).to(BF16).float()
    q = torch.randn(n_rows, hq * hd, generator=g) * 0.05
    q.view(n_rows, hq, hd)[:, :, 0] = 8.0
    return keys, vals, q.to(BF16), 56.0 / (8.0 * scale), scale


@pytest.mark.parametrize("hq", [7, 8])
@pytest.mark.parametrize("n", [16384, 32768, 32768 + 77])
def test_attention_decode_over_tens_of_thousands_of_keys(hq, n):
    from sonicboom_amd import ops
    from sonicboom_amd.cache import layout
    hkv, hd = 1, 128
    keys, vals, q, rise, scale = looking_along_zero(n, hq, hkv, hd, 1, seed=n + hq)
    kc, vc, table = paged(keys, vals, seed=hq)
    pos = torch.tensor([n - 1], dtype=torch.int32, device=DEV)
    # random data: every key counts a little
    qr = torch.randn(1, hq * hd, generator=torch.Generator().manual_seed(1)).to(BF16)
    kr = torch.randn(n, hkv, hd, generator=torch.Generator().manual_seed(2)).to(BF16).float()
    krc, vrc, _ = paged(kr, vals, seed=hq)
    got = ops.attention_decode_mfma(qr.to(DEV), krc, vrc, table.to(DEV), pos, hq, hkv, hd, scale, 0)
    want = plain.attention(qr.float().numpy(), kr.reshape(n, -1).numpy(), vals.reshape(n, -1).numpy(), [n - 1],
                           np.arange(n), hq, hkv, hd, scale)
    close(got, want, atol=1.5e-2, rtol=1e-2, what=f"decode over {n} random keys")
    # one dominant key at a time: the first chunk, a middle one, the last
    for far in (0, 63, n // 2 + 3, n // 2 + 64 * 5 - 1, n - 64 * 3, n - 2, n - 1):
        page, slot = int(table[0, far // 64]), far % 64
        at = int(layout.key_positions(hd)[slot, 0])
        before = kc[page, :, slot, at].clone()
        kc[page, :, slot, at] = rise
        got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos, hq, hkv, hd, scale, 0)
        kc[page, :, slot, at] = before
        close(got, vals[far].repeat_interleave(hq, dim=0).reshape(1, -1).numpy(), atol=2e-2, rtol=1e-2,
              what=f"dominant key at {far} of {n}")


@pytest.mark.parametrize("pages", [1, 2])
@pytest.mark.parametrize("window", [1000, 9000])
def test_attention_decode_window_edge_in_a_far_chunk(window, pages):
    """A window over a row of 20,000 keys cut into some eighty to a hundred and sixty chunks: the
    chunks before the window's first are never written and must not be read as results, the
    window's first key must count and the key before it must not, and the position lies in a
    chunk that is not full.  (The second kernel, which merges the chunks, takes them in rounds
    when they are many; the window starts in a later round than the first.)"""
    from sonicboom_amd import ops
    hq, hkv, hd, n = 6, 2, 128, 20000
    keys, vals, q, rise, scale = looking_along_zero(n, hq, hkv, hd, 1, seed=61)
    group = hq // hkv
    for p in (n - 1, 19000):
        for inside in (False, True):
            k = keys.clone()
            edge = p - window + (1 if inside else 0)
            k[edge, :, 0] = rise
            kc, vc, table = paged(k, vals, seed=5)
            pos = torch.tensor([p], dtype=torch.int32, device=DEV)
            with ops.attention_decode_pages_per_wave(hd, pages):
                got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos, hq, hkv, hd, scale, window)
            if inside:
                want = vals[edge].repeat_interleave(group, dim=0).reshape(1, -1).numpy()
            else:
                want = plain.attention(q.float().numpy(), k.reshape(n, -1).numpy(), vals.reshape(n, -1).numpy(), [p],
                                       np.arange(n), hq, hkv, hd, scale, causal=True, window=window)
                assert np.abs(want - vals[edge].repeat_interleave(group, dim=0).reshape(1, -1).numpy()).max() > 0.5
            close(got, want, atol=2e-2, rtol=1e-2, what=f"position {p}, window {window}, key {edge}")


@pytest.mark.parametrize("height", [16, 32])
@pytest.mark.parametrize("hq", [7, 8])
@pytest.mark.parametrize("n", [16384, 32768])
def test_attention_prefill_over_tens_of_thousands_of_keys(hq, n, height):
    """The last 20 rows of a sequence of n tokens whose earlier keys are cached (what the second
    portion of a long prompt does), and four rows near the start."""
    from sonicboom_amd import ops
    from sonicboom_amd.cache import layout
    hkv, hd = 1, 128
    positions = [0, 1, 70, 200] + list(range(n - 20, n))
    keys, vals, q, rise, scale = looking_along_zero(n, hq, hkv, hd, len(positions), seed=3 * n + hq)
    # the keys that dominate: one in the first page, one in the middle, one that only the last rows see
    far = (5, n // 2 + 3, n - 10)
    for f in far:
        keys[f, :, 0] = rise
    kc, vc, table = paged(keys, vals, seed=11 + hq)
    assert ops.attention_row_tiles(hq, hkv, hd) == (16, 32)
    pos = torch.tensor(positions, dtype=torch.int32)
    tiles = [(r, 1, 0, 0) for r in range(4)] + [(4 + r0, min(height, 20 - r0), 0, 0) for r0 in range(0, 20, height)]
    tiles = torch.tensor(tiles, dtype=torch.int32)
    got = ops.attention_prefill_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), tiles.to(DEV), hq, hkv, hd, scale,
                                     0, tile_rows=height)
    want = plain.attention(q.float().numpy(), keys.reshape(n, -1).numpy(), vals.reshape(n, -1).numpy(), positions,
                           np.arange(n), hq, hkv, hd, scale)
    close(got, want, atol=2e-2, rtol=1e-2, what=f"prefill rows over {n} keys")
    # and what the dominant keys must give, whatever the plain implementation says: the raised keys
    # tie, so a row's output is the mean of the values of those it sees
    def row(i):
        return got[i].float().cpu().reshape(hq, hd)
    assert torch.allclose(row(2), vals[5].expand(hq, hd), atol=2e-2, rtol=1e-2)                    # position 70
    two = (vals[5] + vals[n // 2 + 3]) / 2
    assert torch.allclose(row(4), two.expand(hq, hd), atol=3e-2, rtol=2e-2)                        # position n - 20
    three = (vals[5] + vals[n // 2 + 3] + vals[n - 10]) / 3
    assert torch.allclose(row(-1), three.expand(hq, hd), atol=3e-2, rtol=2e-2)                     # position n - 1


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_rotation_at_positions_of_tens_of_thousands(dtype):
    """The angle is float(position) * inv_freq in 32-bit: at position 131,071 a pair of the first
    frequency has turned 20,860 times, and a float32 sine of such an angle must still be the one
    the plain implementation takes."""
    from sonicboom_amd import ops
    from sonicboom_amd.cache import layout
    hq, hkv, hd, base = 4, 2, 128, 1e6
    pos = torch.tensor([32767, 131071, 65536, 99999, 0, 16384], dtype=torch.int32)
    n = len(pos)
    qkv = torch.randn(n, (hq + 2 * hkv) * hd, generator=torch.Generator().manual_seed(4))
    table = torch.arange(2048, dtype=torch.int32).reshape(1, 2048)       # page = position / 64
    kc = torch.zeros((2048, hkv, 64, hd), dtype=dtype, device=DEV)
    vc = torch.zeros((2048, hkv, hd, 64), dtype=dtype, device=DEV)
    log_base = np.log(np.float32(base)).astype(np.float32)
    inv = np.exp((np.float32(-2.0) * np.arange(hd // 2, dtype=np.float32) / np.float32(hd)).astype(np.float32)
                 * log_base).astype(np.float32)
    seq = torch.zeros(n, dtype=torch.int32)
    q = ops.rope_kv_store(qkv.to(DEV), dtype, torch.from_numpy(inv).to(DEV), None, hd, pos.to(DEV), seq.to(DEV), kc, vc,
                          table.to(DEV), hq, hkv, hd)
    want_q = plain.rope_neox(qkv[:, :hq * hd].numpy(), pos.numpy(), hd, base)
    want_k = plain.rope_neox(qkv[:, hq * hd:(hq + hkv) * hd].numpy(), pos.numpy(), hd, base)
    tol = dict(atol=4e-6, rtol=1e-5) if dtype == F32 else dict(atol=2e-2, rtol=8e-3)
    close(q, want_q, what="q", **tol)
    for r in range(n):
        got_k = layout.get_key(kc, int(pos[r]) // 64, int(pos[r]) % 64).reshape(-1)
        close(got_k, want_k[r], what=f"k at position {int(pos[r])}", **tol)


LONG = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "intermediate_size": 160, "vocab_size": 300, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 32768, "tie_word_embeddings": False, "use_sliding_window": False,
    "hidden_act": "silu",
}


@pytest.fixture(scope="module")
def long_case(tmp_path_factory):
    """A folder of the model above with sharpened queries and keys (scores of several units, so
    that far keys matter), a prompt of 20,000 tokens and the plain logits at its last 8 places."""
    from conftest import sharpen_model
    from sonicboom_amd.weights import write_random_model
    plain_folder, folder = str(tmp_path_factory.mktemp("long_plain")), str(tmp_path_factory.mktemp("long"))
    write_random_model(plain_folder, dict(LONG), seed=99, dtype="bfloat16")
    sharpen_model(plain_folder, folder)
    tokens = random_prompt(np.random.default_rng(20), LONG["vocab_size"], 20000)
    cfg, w = plain.load_model(folder)
    want = plain.forward(cfg, w, tokens)[-8:]
    return folder, tokens, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_20000_tokens(long_case, dtype):
    """More rows than a step takes at once: two portions, the second over the 16,384 keys the first
    left (in bfloat16 both in tiles of 32 rows, the prefill kernel's form for long prompts); then
    the last 8 tokens once more one by one on a second slot (decode over 19,992 keys)."""
    from sonicboom_amd.engine import DecoderModel, Engine, StepEntry
    folder, tokens, want = long_case
    eng = Engine(DecoderModel.from_folder(folder, dtype), 64 * 640)
    assert len(tokens) > eng.max_step_rows
    if dtype == "bfloat16":
        from sonicboom_amd import ops
        assert eng.model.row_tiles == [16, 32] and len(tokens) // 32 >= ops.TALL_MIN_BLOCKS
    s = eng.alloc_slot()
    got = eng.step([StepEntry(s, tokens, range(len(tokens) - 8, len(tokens)))]).cpu().numpy()
    assert_logits_close(got, want, dtype, "the last 8 places of 20,000", sharp=True)
    eng.free_slot(s)
    s = eng.alloc_slot()
    eng.step([StepEntry(s, tokens[:-8], ())])
    rows = [eng.step([StepEntry(s, [t], [0])]).cpu().numpy() for t in tokens[-8:]]
    assert_logits_close(np.concatenate(rows), want, dtype, "the last 8 tokens one by one", sharp=True)
    eng.free_slot(s)
