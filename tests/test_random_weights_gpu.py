"""Random weights: a seed means one model, whether it is drawn on the GPU or on the host, in
memory or into a folder; the load-time kernels (fill, cast and place) against numpy and torch;
and the command line's two ways into the in-memory model (--random, RBITNET_TOY=1)."""
import json
import os
import subprocess
import sys

import pytest
import torch

from helpers import CONFIGS, TINY_A, TINY_B, interleave_gate_up, tokens_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from rbitnet_amd.csrc.lib import kernels
    return kernels()


@pytest.mark.parametrize("n", [1, 2, 7, 4096, 1_000_003])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fill_kernel_equals_its_host_twin_bit_for_bit(lib, n, dtype):
    from rbitnet_amd.weights.random_init import normal_values, tensor_key
    for name, mean, std in (("a.weight", 0.0, 0.02), ("b.norm", 1.0, 0.1)):
        key = tensor_key(7, name)
        out = torch.full((n,), float("nan"), dtype=dtype, device=DEV)
        lib.fill_normal(out, key, mean, std)
        want = torch.from_numpy(normal_values(key, n, mean, std)).to(dtype)
        got = out.cpu()
        same = got.view(torch.int32 if dtype == torch.float32 else torch.int16) == \
            want.view(torch.int32 if dtype == torch.float32 else torch.int16)
        assert bool(same.all()), f"{int((~same).sum())} of {n} values differ"


def test_fill_kernel_draws_normal_numbers(lib):
    from rbitnet_amd.weights.random_init import tensor_key
    out = torch.empty(4_000_000, dtype=torch.float32, device=DEV)
    lib.fill_normal(out, tensor_key(3, "w"), 0.0, 1.0)
    v = out.double()
    assert abs(float(v.mean())) < 4 / 2000 and abs(float(v.std()) - 1) < 3e-3
    assert abs(float((v ** 3).mean())) < 0.02 and abs(float((v ** 4).mean()) - 3) < 0.05       # skew, kurtosis
    assert abs(float((v.abs() > 1.959964).double().mean()) - 0.05) < 1e-3                    # the tails' weight
    even, odd = v[0::2], v[1::2]                          # cosine and sine of a pair are uncorrelated
    assert abs(float((even * odd).mean())) < 3e-3 and abs(float((v[:-1] * v[1:]).mean())) < 3e-3
    gains = torch.empty(100_000, dtype=torch.float32, device=DEV)
    lib.fill_normal(gains, tensor_key(3, "g"), 1.0, 0.02)
    assert abs(float(gains.mean()) - 1) < 3e-4 and abs(float(gains.std()) - 0.02) < 3e-4
    other = torch.empty(100_000, dtype=torch.float32, device=DEV)
    lib.fill_normal(other, tensor_key(3, "h"), 1.0, 0.02)
    assert not torch.equal(other, gains)                  # another name, other numbers


def test_place_rows_casts_and_places(lib):
    g = torch.Generator().manual_seed(0)
    a, b = torch.randn(48, 40, generator=g), torch.randn(48, 40, generator=g)
    for src_dtype, dst_dtype in ((torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32),
                                 (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32)):
        x, y = a.to(src_dtype), b.to(src_dtype)
        # one after the other
        dst = torch.full((100, 40), float("nan"), dtype=dst_dtype, device=DEV)
        lib.place_rows(x.to(DEV), dst, row0=0)
        lib.place_rows(y.to(DEV), dst, row0=48)
        want = torch.cat([x, y]).to(dst_dtype)
        assert torch.equal(dst[:96].cpu(), want) and bool(torch.isnan(dst[96:].float()).all())
        # interleaved in blocks of 16
        dst = torch.full((96, 40), float("nan"), dtype=dst_dtype, device=DEV)
        lib.place_rows(x.to(DEV), dst, row0=0, block=16, period=32)
        lib.place_rows(y.to(DEV), dst, row0=16, block=16, period=32)
        assert torch.equal(dst.cpu(), interleave_gate_up(x, y).to(dst_dtype))
    from rbitnet_amd.errors import KernelError
    with pytest.raises(KernelError, match="beyond"):
        lib.place_rows(a.to(DEV), torch.empty((60, 40), device=DEV), row0=20)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_a_seed_means_one_model_in_memory_and_on_disk(name, dtype, tmp_path):
    """Engine.random(config, seed) and Engine.load_path(write_random_model(config, seed)): the
    same logits bit for bit (the folder is drawn by the host twin, the engine's weights by the
    kernel), and another seed gives another model."""
    import rbitnet_amd
    cfg, seed, norm_std = CONFIGS[name]
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    folder = rbitnet_amd.write_random_model(str(tmp_path / "m"), cfg, seed=seed, std=0.1, norm_std=norm_std,
                                            dtype=store, device="cpu")
    on_disk = rbitnet_amd.Engine.load_path(folder, dtype=dtype, max_tokens=256)
    in_memory = rbitnet_amd.Engine.random(cfg, seed=seed, dtype=dtype, std=0.1, norm_std=norm_std, max_tokens=256)
    other = rbitnet_amd.Engine.random(cfg, seed=seed + 1, dtype=dtype, std=0.1, norm_std=norm_std, max_tokens=256)
    toks = tokens_for(name, 70, 0)
    out = []
    for eng in (on_disk, in_memory, other):
        slot = eng.alloc_slot()
        out.append(torch.cat([eng.step([(slot, toks[:60])], "all")] +
                             [eng.step([(slot, [t])], "last") for t in toks[60:]]).cpu())
        eng.free_slot(slot)
    assert torch.equal(out[0], out[1])
    assert not torch.allclose(out[0], out[2], atol=1e-3)
    # and it is the model that the plain implementation reads from the folder
    from helpers import TOL, max_err
    from plain_llama import PlainLlama
    assert max_err(out[1], PlainLlama.from_folder(folder).logits(toks)) < TOL[dtype]


def _cli(args, env=None, expect=0):
    full_env = dict(os.environ)
    for k in ("RBITNET_TOY", "RBITNET_TOY_SEED", "RBITNET_MODEL"):
        full_env.pop(k, None)
    full_env.update(env or {})
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "rbitnet")] + args, capture_output=True, text=True,
                       env=full_env, timeout=300)
    assert r.returncode == expect, r.stderr[-2000:]
    return r


def test_command_line_random_weights_and_toy_mode(tmp_path):
    """`--random --config`, RBITNET_TOY=1 (seed from RBITNET_TOY_SEED, default 42) and a folder
    written by `rbitnet random` with the same seed: one model, so the same greedy tokens."""
    cfg_path = str(tmp_path / "config.json")
    with open(cfg_path, "w") as f:
        json.dump(TINY_B, f)
    common = ["--prompt-ids", "5,6,7,300", "--prompt-ids", "9", "--max-tokens", "12", "--temperature", "0",
              "--dtype", "float32"]

    def tokens(r):
        return [json.loads(line)["tokens"] for line in r.stdout.strip().splitlines()]

    a = tokens(_cli(["generate", "--random", "--config", cfg_path, "--weight-seed", "42"] + common))
    b = tokens(_cli(["generate", "--config", cfg_path] + common, env={"RBITNET_TOY": "1"}))
    c = tokens(_cli(["generate", "--config", cfg_path] + common, env={"RBITNET_TOY": "1", "RBITNET_TOY_SEED": "43"}))
    folder = str(tmp_path / "m")
    _cli(["random", "--config", cfg_path, "--out", folder, "--seed", "42", "--dtype", "float32"])
    d = tokens(_cli(["generate", "--model", folder] + common))
    assert len(a) == 2 and all(len(t) <= 12 for t in a)
    assert a == b == d and a != c
    # the plain implementation on the written folder generates the same tokens
    from plain_llama import PlainLlama, greedy_generate
    plain = PlainLlama.from_folder(folder)
    stop = (TINY_B["eos_token_id"],)
    assert a == [greedy_generate(plain, [5, 6, 7, 300], 12, stop), greedy_generate(plain, [9], 12, stop)]
    r = _cli(["generate", "--random"] + common, expect=1)
    assert "need --config" in r.stderr


def test_command_line_add_bos(tmp_path):
    """--add-bos puts the configuration's BOS id before every prompt: the same tokens as the prompt
    given with that id in front; a configuration without one refuses the flag."""
    cfg = dict(TINY_B, bos_token_id=11)
    cfg_path = str(tmp_path / "config.json")
    with open(cfg_path, "w") as f:
        json.dump(cfg, f)
    common = ["generate", "--random", "--config", cfg_path, "--max-tokens", "6", "--temperature", "0", "--dtype", "float32"]
    with_flag = [json.loads(line) for line in
                 _cli(common + ["--add-bos", "--prompt-ids", "5,6", "--prompt-ids", "9"]).stdout.strip().splitlines()]
    by_hand = [json.loads(line) for line in
               _cli(common + ["--prompt-ids", "11,5,6", "--prompt-ids", "11,9"]).stdout.strip().splitlines()]
    assert with_flag == by_hand and [r["prompt_tokens"] for r in with_flag] == [3, 2]
    without = [json.loads(line) for line in _cli(common + ["--prompt-ids", "5,6", "--prompt-ids", "9"]).stdout.strip().splitlines()]
    assert [r["prompt_tokens"] for r in without] == [2, 1]
    none = {k: v for k, v in TINY_B.items() if k != "bos_token_id"}
    with open(cfg_path, "w") as f:
        json.dump(none, f)
    r = _cli(common + ["--add-bos", "--prompt-ids", "5"], expect=1)
    assert "bos_token_id" in r.stderr


def test_kernel_times_behind_an_environment_flag(tmp_path):
    """RBITNET_KERNEL_TIMES=1: a table of GPU time per kernel wrapper on standard error when the
    process ends; the tokens are the ones a run without it generates."""
    cfg_path = str(tmp_path / "config.json")
    with open(cfg_path, "w") as f:
        json.dump(TINY_A, f)
    args = ["generate", "--random", "--config", cfg_path, "--prompt-ids", "1,2,3", "--max-tokens", "5", "--temperature", "0"]
    plain = _cli(args)
    timed = _cli(args, env={"RBITNET_KERNEL_TIMES": "1"})
    assert timed.stdout == plain.stdout
    table = timed.stderr
    assert "total ms" in table and "sample" in table and "add_rmsnorm" in table
    calls = {line.split()[0]: int(line.split()[1]) for line in table.splitlines() if line.startswith(("sample", "embed_gather"))}
    assert calls["sample"] == 5 and calls["embed_gather"] == 5        # a prompt step and four decode steps
    assert "total ms" not in plain.stderr
