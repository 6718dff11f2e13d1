"""Host bookkeeping of Mi355Engine.TensorMatMulCachedB (the mirror of SimdGemm.SgemmWithCachedB's PrePackedB cache,
src/AiDotNet.Tensors/Engines/Simd/SimdGemm.cs:292, 327-684): a packed weight belongs to ONE weight tensor.  The reference keys
on array identity through a ConditionalWeakTable; a device address is not an identity, because the allocator hands a freed
block to the next tensor of the same size.  Runs without a GPU: the backend is replaced by a stand-in that "packs" by copying,
so a stale pack shows up as the product of the wrong weight."""
import gc

import torch

from aidotnet.tensors_amd.engine import Mi355Engine


class _CopyingBackend:
    def __init__(self):
        self.packs = 0

    def WrapTensor(self, t):
        return t

    def PackB(self, kind, B, K, N):
        self.packs += 1
        return B.clone()

    def GemmPackedB(self, kind, A, packed, bias, C, M, N, K, outputIsFp32=True):
        C.copy_((A.reshape(M, K) @ packed).reshape(C.shape))


def _engine():
    eng = Mi355Engine.__new__(Mi355Engine)
    eng.backend = _CopyingBackend()
    return eng


def test_a_freed_weight_does_not_leave_its_pack_to_the_next_tensor_at_that_address():
    eng = _engine()
    x = torch.arange(12, dtype=torch.float32).reshape(3, 4)
    for rep in range(8):                       # the allocator returns the block just freed: same address, version 0, same shape
        w = torch.full((4, 5), float(rep + 1))
        got = eng.TensorMatMulCachedB(x, w)
        assert torch.equal(got, x @ w), rep
        del w
        gc.collect()
    assert len(eng._packed_b) == 0             # every entry left with its weight


def test_same_live_weight_is_packed_once_and_a_changed_one_again():
    eng = _engine()
    x = torch.ones(2, 4)
    w = torch.ones(4, 3)
    eng.TensorMatMulCachedB(x, w); eng.TensorMatMulCachedB(x, w)
    assert eng.backend.packs == 1
    w.mul_(3)
    assert torch.equal(eng.TensorMatMulCachedB(x, w), x @ w) and eng.backend.packs == 2


def test_transposed_views_are_never_served_from_another_weights_pack():
    eng = _engine()
    x = torch.arange(8, dtype=torch.float32).reshape(2, 4)
    w1 = torch.arange(20, dtype=torch.float32).reshape(5, 4)
    w2 = -w1
    assert torch.equal(eng.TensorMatMulCachedB(x, w1.t()), x @ w1.t())
    assert torch.equal(eng.TensorMatMulCachedB(x, w2.t()), x @ w2.t())
    assert len(eng.__dict__.get("_packed_b", {})) == 0      # temporary contiguous copies are not cached


def test_capacity_bound_drops_the_least_recently_used_weight():
    eng = _engine()
    eng.CACHED_B_CAPACITY = 2
    x = torch.ones(1, 2)
    ws = [torch.full((2, 2), float(i)) for i in range(3)]
    for w in ws:
        eng.TensorMatMulCachedB(x, w)
    assert len(eng._packed_b) == 2 and id(ws[0]) not in eng._packed_b
