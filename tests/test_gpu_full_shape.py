"""The verify-step driver at the headline benchmark's full shape (48 layers = 12 x (3 GatedDelta + 1 attention),
Qwen3-Next head shapes, 32K context): what the steps leave in the buffers is checked against float64 / float32
restatements written in torch (bench.StepChecker, the same checks bench.py runs after its timed region), and a
HIP-graph replay of the steps is compared with eager stepping byte for byte."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _stack(seed=0, **kw):
    from swiftlm_amd.verify_step import HybridVerifyStack, StackConfig

    return HybridVerifyStack(StackConfig(max_steps=8, **kw), seed=seed)


def test_config4_full_shape_steps_match_restatements(gpu_lib):
    from bench import StepChecker

    stack = _stack()
    cfg = stack.cfg
    assert (cfg.n_layers, cfg.context, cfg.Hv, cfg.Dk, cfg.Hq, cfg.Hkv, cfg.D) == (48, 32768, 32, 128, 16, 2, 256)
    offset = cfg.context
    for step, cc in enumerate([4, 16, 1]):                 # partial acceptance, full acceptance, nothing accepted
        checker = StepChecker(stack, gdn_layers=(0, 17, 35), attn_layers=(0, 11))
        ph = stack.phase
        stack.set_acceptance(ph, cc, seed=step)
        posterior = stack.posterior[ph].cpu()
        stack.enqueue_step()
        torch.cuda.synchronize()
        offset += cc
        assert int(stack.offset) == offset
        errs = checker.check([cc], [posterior])
        assert errs and all(v == v for v in errs.values())


def test_config4_two_steps_chain_in_one_check(gpu_lib):
    """Two steps between snapshot and check, as bench.py's post-timing check runs them."""
    from bench import StepChecker

    stack = _stack(seed=1)
    checker = StepChecker(stack, gdn_layers=(5,), attn_layers=(3,))
    posts = []
    for step, cc in enumerate([7, 2]):
        ph = stack.phase
        stack.set_acceptance(ph, cc, seed=10 + step)
        posts.append(stack.posterior[ph].cpu())
        stack.enqueue_step()
    torch.cuda.synchronize()
    checker.check([7, 2], posts)


def test_config4_graph_replay_equals_eager_stepping(gpu_lib):
    """The same token ids through a captured graph (two steps per graph, as bench.py times them) and through eager
    calls leave identical bytes everywhere: states, tapes, y, attention outputs, logsumexp, offsets, accept words."""
    eager, graphed = _stack(seed=2), _stack(seed=2)
    commits = [4, 16, 1, 7]
    T = eager.cfg.block

    # ids of all four steps, staged on the device as [step, ids | posterior, T]
    staged = []
    for step, cc in enumerate(commits):
        eager.set_acceptance(0, cc, seed=step)
        staged.append(eager.accept_inputs[0].clone())
    staged = torch.stack(staged)

    for step in range(4):
        eager.accept_inputs[eager.phase].copy_(staged[step])
        eager.enqueue_step()
    torch.cuda.synchronize()

    # the second stack only ever runs through the graph (the eager stack above has already loaded every code object,
    # so nothing is set up inside the capture)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    assert graphed.phase == 0
    with torch.cuda.graph(g, stream=side):
        graphed.enqueue_step()
        graphed.enqueue_step()
    torch.cuda.current_stream().wait_stream(side)
    assert graphed.phase == 0
    for pair in range(2):
        graphed.accept_inputs.copy_(staged[2 * pair:2 * pair + 2])
        g.replay()
        torch.cuda.synchronize()           # the program's own synchronisation between replays
    assert int(eager.offset) == int(graphed.offset) == eager.cfg.context + sum(commits)
    assert eager.accept.tolist() == graphed.accept.tolist()
    assert eager.phase == graphed.phase == 0
    for a, b in zip(eager.gdn, graphed.gdn):
        assert torch.equal(a["state"][0], b["state"][0]) and torch.equal(a["state"][1], b["state"][1])
        assert torch.equal(a["tape"], b["tape"]) and torch.equal(a["y"], b["y"])
    n = int(eager.offset) + T
    for a, b in zip(eager.attn, graphed.attn):
        assert torch.equal(a["out"], b["out"]) and torch.equal(a["lse"], b["lse"])
        assert torch.equal(a["k_cache"][:, :, :n], b["k_cache"][:, :, :n])
        assert torch.equal(a["v_cache"][:, :, :n], b["v_cache"][:, :, :n])


def test_config4_sixty_four_consecutive_steps(gpu_lib):
    """The benchmark configuration's full run: 64 consecutive verify steps at the full shape, accepted lengths drawn
    Geometric(0.25) in [1, 16] as the benchmark draws them, stepped the way the benchmark times them (eight steps per
    captured graph, eight launches).  After the 64th step: cache offset, accept words and the rows every step appended
    bit-exact; the recurrent state of three GatedDelta layers against the float64 recurrence over exactly the tokens
    the 64 steps committed (rtol 1e-4); tape, y and the attention outputs of the last step against their restatements."""
    from bench import StepChecker, draw_commit_counts
    from swiftlm_amd.verify_step import HybridVerifyStack, StackConfig

    steps, per_graph = 64, 8
    stack = HybridVerifyStack(StackConfig(max_steps=steps + 2), seed=4, n_slots=per_graph)
    T = stack.cfg.block
    commits = draw_commit_counts(steps, T, seed=99)
    assert 1 in commits and max(commits) > 8
    commits[5] = T                                           # a fully accepted block (no replay) is part of the run
    staged, posts = [], []
    for s, cc in enumerate(commits):
        stack.set_acceptance(0, cc, seed=s)
        staged.append(stack.accept_inputs[0].clone())
        posts.append(stack.posterior[0].cpu())
    staged = torch.stack(staged)
    # one eager step on a scratch stack first, so that nothing is set up inside the capture
    HybridVerifyStack(StackConfig(max_steps=2, n_layers=8), seed=0).enqueue_step()
    torch.cuda.synchronize()
    checker = StepChecker(stack, gdn_layers=(0, 17, 35), attn_layers=(0, 11))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        for i in range(per_graph):
            stack.enqueue_step(slot=i)
    torch.cuda.current_stream().wait_stream(side)
    assert stack.phase == 0
    for r in range(steps // per_graph):
        stack.accept_inputs[:per_graph].copy_(staged[r * per_graph:(r + 1) * per_graph])
        g.replay()
        torch.cuda.synchronize()
    assert int(stack.offset) == stack.cfg.context + sum(commits)
    errs = checker.check(commits, posts)
    assert errs and all(v == v for v in errs.values())
