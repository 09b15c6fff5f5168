"""Steps whose launches are issued from C++ (engine/step_plan.py): a shape that comes back is
recorded and then replayed; every replay gives what the same step gives launched from Python, bit
for bit, whatever was allocated or computed in between, and what the plain implementation gives."""
import pytest
import torch

from helpers import TOL, max_err, model_folder, plain_logits, tokens_for

pytestmark = pytest.mark.gpu


def _engine(name, dtype, **kw):
    import rbitnet_amd
    kw.setdefault("max_tokens", 2048)
    return rbitnet_amd.Engine.load_path(model_folder(name), dtype=dtype, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_replayed_steps_equal_steps_launched_from_python(name, dtype):
    eager, planned = _engine(name, dtype, max_batch=4), _engine(name, dtype, max_batch=4)
    eager.use_plans = False
    assert planned.use_plans
    lengths = [70, 5, 33]
    junk = []
    for round_ in range(4):                       # the same shapes four times with other tokens: seen, recorded, replayed twice
        reqs = [tokens_for(name, n + 4, 100 * round_ + i) for i, n in enumerate(lengths)]
        outs = []
        for eng in (eager, planned):
            for g in eng.cache.kv_groups:
                g.k.fill_(float("nan"))
                g.v.fill_(float("nan"))
            slots = [eng.alloc_slot() for _ in reqs]
            got = [eng.step([(s, r[:n]) for s, r, n in zip(slots, reqs, lengths)], "all")]
            for j in range(4):
                got.append(eng.step([(s, [r[n + j]]) for s, r, n in zip(slots, reqs, lengths)], "last"))
                if eng is planned:                # unrelated allocations and work between the steps
                    junk.append(torch.randn(1000 + 37 * len(junk), device="cuda"))
                    _ = (junk[-1] * 2).sum().item()
            for s in slots:
                eng.free_slot(s)
            outs.append(got)
        for a, b in zip(*outs):
            assert torch.equal(a, b), f"round {round_}"
        off = 0
        for i, (r, n) in enumerate(zip(reqs, lengths)):
            want = plain_logits(name, tuple(r))
            assert max_err(outs[1][0][off:off + n], want[:n]) < TOL[dtype]
            off += n
            tail = torch.cat([outs[1][1 + j][i:i + 1] for j in range(4)])
            assert max_err(tail, want[n:n + 4]) < TOL[dtype]
    # the prompt step once and each of the four single-token steps' shape once (they differ in nothing
    # that the key holds unless a page table grows): recorded in round 1, replayed in rounds 2 and 3
    stats = planned.plans.stats
    assert stats["recorded"] >= 2 and stats["replayed"] >= 2 * stats["recorded"]
    assert eager.plans.stats == {"recorded": 0, "replayed": 0}
    planned.cache.check()


def test_a_shape_seen_once_is_not_recorded_and_old_plans_make_room():
    from rbitnet_amd.engine import step_plan
    eng = _engine("A", "float32", max_batch=1, max_tokens=256)
    slot = eng.alloc_slot()
    eng.step([(slot, tokens_for("A", 9, 1))], "last")
    assert eng.plans.stats == {"recorded": 0, "replayed": 0} and len(eng.plans.plans) == 0
    eng.free_slot(slot)
    for n in range(1, step_plan.MAX_PLANS + 4):                 # more shapes than are kept
        for _ in range(2):
            slot = eng.alloc_slot()
            eng.step([(slot, tokens_for("A", n, n))], "last")
            eng.free_slot(slot)
    assert len(eng.plans.plans) == step_plan.MAX_PLANS
    assert eng.plans.stats["recorded"] == step_plan.MAX_PLANS + 3
    want = plain_logits("A", tuple(tokens_for("A", 2, 77)))
    slot = eng.alloc_slot()
    assert max_err(eng.step([(slot, tokens_for("A", 2, 77))], "last"), want[-1:]) < TOL["float32"]
    assert eng.plans.stats["recorded"] == step_plan.MAX_PLANS + 4          # recorded anew, the oldest being gone
    eng.free_slot(slot)


def test_a_model_with_a_part_of_its_own_runs_without_plans():
    """A part that computes with torch operations is not `plan_safe`: nobody would issue those again."""
    import rbitnet_amd
    from rbitnet_amd.config.spec import LayerSpec, ModelSpec, PartSpec
    from rbitnet_amd.engine.model import expected_tensors
    from rbitnet_amd.parts import Part, TensorSpec, register_feed_forward
    from rbitnet_amd.weights import random_tensors

    class Doubling(Part):
        graph_safe = True

        def __init__(self, params, env):
            self.env = env

        def forward(self, h, ctx=None):
            return h.float() * 2.0

    register_feed_forward("doubling_for_tests", Doubling)
    norm = PartSpec("rmsnorm", {"size": 32, "eps": 1e-5})
    att = {"num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "scale": 0.25, "window": None, "cache_from": None,
           "position": PartSpec("rope", {"head_dim": 16, "theta": 100.0, "max_positions": 128})}
    spec = ModelSpec(architecture="ToyForTests", hidden_size=32, vocab_size=50, max_positions=128,
                     layers=[LayerSpec("blocks.0", "prenorm", PartSpec("attention", att),
                                       PartSpec("doubling_for_tests", {}), norm, norm)],
                     embedding_name="embed.weight", final_norm=norm, final_norm_name="final_norm.weight",
                     head_name="head.weight")
    tensors = dict(random_tensors(expected_tensors(spec), seed=1, std=0.1, norm_std=0.0, dtype=torch.bfloat16))
    eng = rbitnet_amd.Engine.from_spec(spec, tensors, dtype="float32", max_tokens=128, max_batch=1)
    assert not eng.use_plans
    slot = eng.alloc_slot()
    a = eng.step([(slot, [1, 2, 3])], "last")
    eng.free_slot(slot)
    slot = eng.alloc_slot()
    assert torch.equal(a, eng.step([(slot, [1, 2, 3])], "last"))
    assert eng.plans.stats == {"recorded": 0, "replayed": 0}
