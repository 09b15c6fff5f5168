"""The kernels that only wide models select (256 x 256 tiles, the token-resident and the
panel products, flash attention over many blocks, decode splits) at the widths of Llama-3-8B
with two layers: the float32 engine against the plain implementation, and the bfloat16
engine's prompt step, decode steps and a mid-size batch against the float32 engine."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

WIDE = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "num_hidden_layers": 2,
    "num_attention_heads": 32, "num_key_value_heads": 8, "intermediate_size": 14336, "vocab_size": 128256,
    "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 1024},
}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    import rbitnet_amd
    path = str(tmp_path_factory.mktemp("wide") / "m")
    # std 0.03: large enough for attention and the gate to matter at this width
    return rbitnet_amd.write_random_model(path, WIDE, seed=5, std=0.03, norm_std=0.05, dtype=torch.bfloat16)


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max())


def test_wide_model_float32_against_plain(folder):
    """The float32 engine at full width (sums over 4,096 and 14,336 terms, a vocabulary of
    128,256) against the plain implementation in float64, whose sums run on the GPU for their
    size: a prompt in one step, then tokens one by one."""
    import os
    import sys
    sys.path.insert(0, os.path.dirname(__file__))
    import rbitnet_amd
    from plain_llama import PlainLlama
    rng = np.random.default_rng(11)
    tokens = [int(t) for t in rng.integers(0, 128256, size=40)]
    plain = PlainLlama.from_folder(folder, device="cuda:0")
    want = plain.logits(tokens).cpu()
    del plain
    torch.cuda.empty_cache()
    eng = rbitnet_amd.Engine.load_path(folder, dtype="float32", max_tokens=64, max_batch=1)
    slot = eng.alloc_slot()
    got = [eng.step([(slot, tokens[:34])], "all")]
    for t in tokens[34:]:
        got.append(eng.step([(slot, [t])], "last"))
    eng.free_slot(slot)
    got = torch.cat(got).cpu()
    assert got.shape == want.shape
    assert _rel(got, want) < 2e-5


def test_wide_model_bfloat16_against_float32(folder):
    import rbitnet_amd
    rng = np.random.default_rng(3)
    lengths = [700, 130, 65, 300, 1, 31, 64, 200, 90, 17, 450, 33, 257, 129, 5, 512, 77, 256, 40, 100]
    prompts = [[int(t) for t in rng.integers(0, 128256, size=n)] for n in lengths]
    tail = 3                                        # tokens of each request that are decoded one by one

    ref = rbitnet_amd.Engine.load_path(folder, dtype="float32", max_tokens=64 * 80, max_batch=len(prompts))
    want = []
    for p in prompts:
        s = ref.alloc_slot()
        rows = list(range(max(0, len(p) - tail - 1), len(p)))
        want.append(ref.step([(s, p)], [rows]).cpu())
        ref.free_slot(s)
    del ref
    torch.cuda.empty_cache()

    eng = rbitnet_amd.Engine.load_path(folder, dtype="bfloat16", max_tokens=64 * 80, max_batch=len(prompts))
    tol = 3e-2
    # (1) each alone: a prompt step (tiled products, flash attention), then single tokens (skinny and
    #     token-resident products, decode attention with splits)
    for p, w in zip(prompts[:6], want[:6]):
        s = eng.alloc_slot()
        head = max(1, len(p) - tail)
        got = [eng.step([(s, p[:head])], "last")]
        for t in p[head:]:
            got.append(eng.step([(s, [t])], "last"))
        eng.free_slot(s)
        got = torch.cat(got).cpu()
        assert _rel(got, w[-got.shape[0]:]) < tol, len(p)
    # (2) all twenty together: one ragged prompt step, then batch-20 steps (panel products) through the
    #     graph path, the requests' last `tail` tokens being fed one by one
    slots = [eng.alloc_slot() for _ in prompts]
    heads = [max(1, len(p) - tail) for p in prompts]
    logits = eng.step([(s, p[:h]) for s, p, h in zip(slots, prompts, heads)], "last").cpu()
    for i, (p, h, w) in enumerate(zip(prompts, heads, want)):
        assert _rel(logits[i:i + 1], w[h - 1 - (len(p) - w.shape[0]):][:1]) < tol, ("prompt", i)
    for j in range(tail):
        live = [i for i, (p, h) in enumerate(zip(prompts, heads)) if h + j < len(p)]
        logits = eng.step([(slots[i], [prompts[i][heads[i] + j]]) for i in live], "last").cpu()
        for r, i in enumerate(live):
            w = want[i]
            pos = heads[i] + j
            assert _rel(logits[r:r + 1], w[pos - (len(prompts[i]) - w.shape[0]):][:1]) < tol, ("decode", i, j)
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()
