"""Boundary behaviour around the library-owned workspace: one workspace per stream (two streams on one context do not race),
blocks that were handed out stay valid after the workspace grows (a captured graph keeps replaying correctly), growth during
capture is refused, the decode entry points refuse descriptors they would otherwise silently ignore, and the packed-weight
form of the MHA forward equals the gathering one."""
import ctypes
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture()
def be():
    from aidotnet.tensors_amd import Mi355Backend
    b = Mi355Backend(synchronous=False)
    yield b
    torch.cuda.synchronize()
    b.Dispose()


def test_two_streams_on_one_context_do_not_share_split_partials(be):
    """Decode attention (split-KV partials) on one stream and the small-M / skinny split-K GEMMs on another, launched back to
    back many times without synchronising: every result must equal the one computed alone."""
    W = be.WrapTensor
    torch.manual_seed(3)
    B, H, S, D = 8, 16, 4096, 128
    q = torch.randn(B, H, 1, D, device="cuda").to(torch.bfloat16)
    k = torch.randn(B, H, S, D, device="cuda").to(torch.bfloat16); v = torch.randn(B, H, S, D, device="cuda").to(torch.bfloat16)
    a32 = torch.randn(4, 4096, device="cuda"); b32 = torch.randn(4096, 4096, device="cuda") * 0.02
    a16 = torch.randn(16, 4096, device="cuda").to(torch.bfloat16); b16 = (torch.randn(4096, 4096, device="cuda") * 0.02).to(torch.bfloat16)
    sc = 1 / math.sqrt(D)

    def decode(o):
        be.DecodeAttention("bf16", W(q), W(k), W(v), W(o), B, H, S, D, sc, 0, 8)

    def gemms(c32, c16):
        be.Gemm(W(a32), W(b32), W(c32), 4, 4096, 4096)
        be.Bf16Gemm(W(a16), W(b16), W(c16), 16, 4096, 4096)

    o_ref = torch.empty(B, H, 1, D, device="cuda"); c32_ref = torch.empty(4, 4096, device="cuda")
    c16_ref = torch.empty(16, 4096, device="cuda", dtype=torch.bfloat16)
    decode(o_ref); gemms(c32_ref, c16_ref); torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    for it in range(12):
        o = torch.zeros_like(o_ref); c32 = torch.zeros_like(c32_ref); c16 = torch.zeros_like(c16_ref)
        with torch.cuda.stream(s1):
            decode(o)
        with torch.cuda.stream(s2):
            gemms(c32, c16)
        outs.append((o, c32, c16))
    torch.cuda.synchronize()
    for it, (o, c32, c16) in enumerate(outs):
        assert torch.equal(o, o_ref), "decode result of round %d changed under a concurrent GEMM" % it
        assert torch.equal(c32, c32_ref) and torch.equal(c16, c16_ref), "GEMM result of round %d changed under a concurrent decode" % it
    with torch.cuda.stream(s1):
        n1 = be.WorkspaceBytes()
    with torch.cuda.stream(s2):
        n2 = be.WorkspaceBytes()
    assert n1 > 0 and n2 > 0


def test_graph_replay_survives_workspace_growth_and_capture_refuses_growth(be):
    from aidotnet.tensors_amd.backend import InvalidOperationException
    W = be.WrapTensor
    torch.manual_seed(4)
    B, H, S, D = 2, 8, 2048, 128
    q = torch.randn(B, H, 1, D, device="cuda").to(torch.bfloat16)
    k = torch.randn(B, H, S, D, device="cuda").to(torch.bfloat16); v = torch.randn(B, H, S, D, device="cuda").to(torch.bfloat16)
    o = torch.empty(B, H, 1, D, device="cuda")
    sc = 1 / math.sqrt(D)
    side = torch.cuda.Stream()

    def step():
        be.DecodeAttention("bf16", W(q), W(k), W(v), W(o), B, H, S, D, sc, 0, 8)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        # nothing has run on this stream: capturing now would have to allocate, which the library refuses
        assert be.WorkspaceBytes() == 0
        be.ReserveWorkspace(1 << 20)
        assert be.WorkspaceBytes() >= (1 << 20)
        step(); torch.cuda.synchronize()
        eager = o.clone()
        with torch.cuda.graph(graph, stream=side):
            step()
        # a larger eager problem on the same stream grows the workspace after the capture ...
        Bb, Hb = 32, 32
        qb = torch.randn(Bb, Hb, 1, D, device="cuda").to(torch.bfloat16)
        kb = torch.randn(Bb, Hb, S, D, device="cuda").to(torch.bfloat16)
        ob = torch.empty(Bb, Hb, 1, D, device="cuda")
        before = be.WorkspaceBytes()
        be.DecodeAttention("bf16", W(qb), W(kb), W(kb), W(ob), Bb, Hb, S, D, sc, 0, 8)
        torch.cuda.synchronize()
        assert be.WorkspaceBytes() > before
    # ... and the graph, which holds the old block's address, still replays correctly
    for it in range(3):
        o.fill_(0); torch.cuda.synchronize()
        graph.replay(); torch.cuda.synchronize()
        assert torch.equal(o, eager), "replay %d after workspace growth differs" % it
    # growth while capturing is refused with a clear error and launches nothing
    other = torch.cuda.Stream()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(other):
        with torch.cuda.graph(g2, stream=other):
            with pytest.raises(InvalidOperationException):
                step()


def test_gemm_under_capture_without_reserved_workspace_takes_the_tiled_kernel(be):
    # a few-row fp32 product and a skinny bf16 product would use split-K partials; on a stream that is being captured and has no
    # workspace yet they run their workspace-free kernels instead of failing, and the replay matches an eager run within tolerance
    W = be.WrapTensor
    torch.manual_seed(9)
    M, N, K = 128, 1024, 4096
    a = torch.randn(M, K, device="cuda"); b = 0.02 * torch.randn(K, N, device="cuda"); c = torch.zeros(M, N, device="cuda")
    a16 = torch.randn(16, K, device="cuda").bfloat16(); b16 = (0.02 * torch.randn(K, N, device="cuda")).bfloat16()
    c16 = torch.zeros(16, N, device="cuda", dtype=torch.bfloat16)
    ref = (a.double() @ b.double()); ref16 = a16.double() @ b16.double()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        assert be.WorkspaceBytes() == 0
        with torch.cuda.graph(graph, stream=side):
            be.Gemm(W(a), W(b), W(c), M, N, K)
            be.Bf16Gemm(W(a16), W(b16), W(c16), 16, N, K)
        assert be.WorkspaceBytes() == 0
    for _ in range(2):
        c.zero_(); c16.zero_(); torch.cuda.synchronize()
        graph.replay(); torch.cuda.synchronize()
        assert float((c.double() - ref).abs().max()) <= 1e-4 * float(ref.abs().max())
        assert float((c16.double() - ref16).abs().max()) <= 2e-2 * float(ref16.abs().max())
    # eager, the same calls take the split paths (the workspace appears) and agree
    be.Gemm(W(a), W(b), W(c), M, N, K); torch.cuda.synchronize()
    assert be.WorkspaceBytes() > 0
    assert float((c.double() - ref).abs().max()) <= 1e-4 * float(ref.abs().max())


def test_decode_refuses_softcap_and_masks(be):
    from aidotnet.tensors_amd._lib import AttnDesc
    t = torch.zeros(4 * 64, device="cuda")
    for kw in ({"softcap": 30.0}, {"mask_mode": 1}):
        d = AttnDesc(B=1, H=4, Hkv=4, Sq=1, Sk=1, D=64, scale=1.0, **kw)
        st = be._lib.aidn_mi355_attn_decode_f32(be._ctx, be._stream(), ctypes.byref(d), t.data_ptr(), t.data_ptr(), t.data_ptr(),
                                                t.data_ptr(), None, 0)
        assert st == 1002
        assert b"soft-cap" in be._lib.aidn_mi355_last_error(be._ctx)


@pytest.mark.parametrize("kind", ["f32", "bf16"])
def test_packed_qkv_weight_gives_the_same_mha_forward(be, kind):
    W = be.WrapTensor
    torch.manual_seed(5)
    dt = torch.float32 if kind == "f32" else torch.bfloat16
    B, S, dM, heads = 2, 96, 256, 4
    x = torch.randn(B, S, dM, device="cuda").to(dt)
    wq, wk, wv, wo = ((0.05 * torch.randn(dM, dM, device="cuda")).to(dt) for _ in range(4))
    y0 = torch.empty(B, S, dM, device="cuda", dtype=dt); y1 = torch.empty_like(y0)
    be.MultiHeadAttentionForward(kind, W(x), W(wq), W(wk), W(wv), W(wo), None, W(y0), B, S, dM, heads)
    packed = be.PackQkvWeights(kind, W(wq), W(wk), W(wv), dM)
    torch.cuda.synchronize()
    assert torch.equal(packed.tensor.view(dt).reshape(dM, 3 * dM), torch.cat([wq, wk, wv], dim=1))
    be.MultiHeadAttentionForwardPacked(kind, W(x), packed, W(wo), None, W(y1), B, S, dM, heads)
    torch.cuda.synchronize()
    assert torch.equal(y0, y1)
