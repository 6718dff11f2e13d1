"""The allocation-free decode entry point (aidn_mi355_attn_decode_bf16_noalloc: split-KV partials in the library's static
device array) against the ordinary entry point, through the C ABI: same kernels, so the outputs must be bit-identical.  Two
calls in a row on the same array, the second with a smaller problem; the oracle bounds the first."""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import mixed_err

pytestmark = pytest.mark.gpu


def _case(be, B, H, Hkv, S, D, splits, seed):
    g = torch.Generator(device="cuda"); g.manual_seed(seed)
    q = torch.randn(B, H, 1, D, device="cuda", generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, S, D, device="cuda", generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, S, D, device="cuda", generator=g).to(torch.bfloat16)
    W = be.WrapTensor
    sc = 1.0 / math.sqrt(D)
    outs = {}
    for no_alloc in (True, False):             # the allocation-free call first: nothing has sized a workspace for it
        o = torch.full((B, H, 1, D), float("nan"), device="cuda")
        lse = torch.full((B, H), float("nan"), device="cuda")
        before = be.WorkspaceBytes()
        be.DecodeAttention("bf16", W(q), W(k), W(v), W(o), B, H, S, D, sc, Hkv, splits, False, W(lse), noAlloc=no_alloc)
        if no_alloc:
            assert be.WorkspaceBytes() == before, "the allocation-free entry point grew the library workspace"
        outs[no_alloc] = (o.cpu().numpy(), lse.cpu().numpy())
    (o0, l0), (o1, l1) = outs[False], outs[True]
    assert np.array_equal(o0, o1) and np.array_equal(l0, l1), "allocation-free entry point differs from the ordinary one"
    return q, k, v, o1, sc


def test_no_alloc_decode_matches_ordinary_entry_point_twice():
    from aidotnet.tensors_amd import Mi355Backend
    from aidotnet.tensors_amd.backend import NotSupportedException
    be = Mi355Backend()
    try:
        # first call: 4 splits of a 2048-key cache; second call: a smaller problem on the same static array
        assert be.WorkspaceBytes() == 0                      # a fresh context holds no workspace
        q, k, v, o, sc = _case(be, 4, 16, 4, 2048, 128, 4, 11)
        want, _ = oracle.attention_f64(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), sc)
        assert mixed_err(o, want) <= 2e-2
        q, k, v, o, sc = _case(be, 2, 8, 8, 600, 64, 2, 12)
        want, _ = oracle.attention_f64(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), sc)
        assert mixed_err(o, want) <= 2e-2
        # partials beyond the static array's 8 MiB are refused and nothing is launched; the buffers are real and correctly sized
        # (one K/V head keeps the cache small), so that a launch, should the size check ever move, stays inside them
        B, H, Hkv, S, D, splits = 16, 64, 1, 4096, 128, 16       # 16 * 64 * 16 * 130 * 4 bytes = 8.1 MiB of partials
        qb = torch.zeros(B, H, 1, D, device="cuda", dtype=torch.bfloat16)
        kb = torch.zeros(B, Hkv, S, D, device="cuda", dtype=torch.bfloat16)
        ob = torch.zeros(B, H, 1, D, device="cuda")
        from aidotnet.tensors_amd._lib import AttnDesc
        import ctypes
        desc = AttnDesc(B=B, H=H, Hkv=Hkv, Sq=1, Sk=S, D=D, scale=sc)
        st = be._lib.aidn_mi355_attn_decode_bf16_noalloc(be._ctx, be._stream(), ctypes.byref(desc), qb.data_ptr(), kb.data_ptr(),
                                                         kb.data_ptr(), ob.data_ptr(), None, splits)
        torch.cuda.synchronize()
        assert st == 1002, st
        with pytest.raises(NotSupportedException):
            be._check(st)
    finally:
        be.Dispose()
