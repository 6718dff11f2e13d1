"""The entry points are launch-only once the workspace of the stream is sized: a decode step (query projection with the rotary
embedding in its summing pass, decode attention, output projection) is captured into a HIP graph and replayed; every replay must
equal the eager result, and the eager result must equal the step with projection and rotation as separate calls.
Between replays the program does its own eager work and synchronises, and the inputs change, so stale-node effects show."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_decode_step_under_hip_graph_matches_eager():
    from aidotnet.tensors_amd import Mi355Backend
    be = Mi355Backend(synchronous=False)
    W = be.WrapTensor
    torch.manual_seed(0)
    B, H, Hkv, D, S, dM = 4, 16, 4, 128, 1024, 2048
    x = torch.randn(B, dM, device="cuda").to(torch.bfloat16)
    wq = (0.02 * torch.randn(dM, H * D, device="cuda")).to(torch.bfloat16)
    wo = (0.02 * torch.randn(H * D, dM, device="cuda")).to(torch.bfloat16)
    kc = torch.randn(B, Hkv, S, D, device="cuda").to(torch.bfloat16); vc = torch.randn(B, Hkv, S, D, device="cuda").to(torch.bfloat16)
    half = D // 2
    ang = torch.arange(S, device="cuda", dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(half, device="cuda") * 2.0 / D))[None, :]
    cos, sin = torch.cos(ang).contiguous(), torch.sin(ang).contiguous()
    q = torch.empty(B, H * D, device="cuda", dtype=torch.bfloat16)
    att = torch.empty(B, H * D, device="cuda", dtype=torch.bfloat16)
    y = torch.empty(B, dM, device="cuda", dtype=torch.bfloat16)

    def step(fused=True):
        if fused:
            # query projection (skinny, split-K) rotated at position S-1 in its summing pass: two launches instead of three
            be.GemmRope("bf16", W(x), W(wq), W(q), B, H * D, dM, W(cos), W(sin), D, H * D, 1, S - 1)
        else:
            be.Bf16Gemm(W(x), W(wq), W(q), B, H * D, dM)
            be.RopeInterleaved(W(q), W(cos), W(sin), W(q), B * H, D, 1, S - 1, "bf16")
        be.DecodeAttention("bf16", W(q), W(kc), W(vc), W(att), B, H, S, D, 1 / math.sqrt(D), Hkv, 0, True)
        be.Bf16Gemm(W(att), W(wo), W(y), B, dM, H * D)                                      # output projection

    step(False); torch.cuda.synchronize()
    unfused = y.clone(); q_unfused = q.clone()
    step(); torch.cuda.synchronize()                      # an eager run: sizes the workspace of the stream it ran on
    eager = y.clone()
    assert torch.equal(q, q_unfused) and torch.equal(eager, unfused)      # same values, rounding included
    need = be.WorkspaceBytes()
    assert need > 0

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        # the workspace is per stream: the capture stream gets its own, reserved before the capture (nothing may be
        # allocated while capturing)
        be.ReserveWorkspace(need)
        with torch.cuda.graph(graph, stream=side):
            step()
    for it in range(4):
        y.fill_(0); att.fill_(0); q.fill_(0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), "replay %d differs from the eager result" % it
        # eager work of the program between replays, and new inputs for the next comparison
        x.copy_(torch.randn(B, dM, device="cuda").to(torch.bfloat16))
        step(); torch.cuda.synchronize()
        eager = y.clone()
