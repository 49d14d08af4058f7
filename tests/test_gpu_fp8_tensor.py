"""GPU test of the FP8 all-gather payload hooks and of the gathered weight in the grouped linear
(gpatch_v4/models/deepseek_v4/fp8_tensor.py:133-244, fp8.py:212-214; the reference runs these on real ranks in
tests/test_gpatch_v4/test_fsdp2_fp8_all_gather.py).  One GPU here: every "rank" is a call of the pre-gather hook on
that rank's shard with a stand-in mesh, and the gather is a concatenation of the payloads in rank order -- which is
what an all-gather delivers.  What is checked: the payload is byte-identical to quantising the whole parameter
(against the CPU oracle), the statistics, the refusal of a wrong shard shape, and that the grouped linear gives
the same output for the gathered weight as for the plain (codes, scales) pair."""
import types

import pytest
import torch

from oracle import torch_ref as T

pytestmark = pytest.mark.gpu


class _Mesh:
    def __init__(self, world, rank):
        self._world, self._rank = world, rank

    def size(self):
        return self._world

    def get_local_rank(self):
        return self._rank


def say(*a):
    print("[case]", *a, flush=True)


def _gather(full, world, module):
    from gcore_lowp.fp8_tensor import Fp8TensorAg
    experts = full.shape[0]
    chunk = -(-experts // world)
    payloads, metas, owners = [], [], []
    for r in range(world):
        shard = full[min(r * chunk, experts):min((r + 1) * chunk, experts)].clone()
        owner = Fp8TensorAg(shard)
        (codes, carrier), meta = owner.fsdp_pre_all_gather(_Mesh(world, r), full.shape, full.stride(), module, None)
        assert codes.dtype == torch.uint8 and carrier.dtype == torch.uint8
        assert tuple(codes.shape) == (chunk,) + tuple(full.shape[1:])
        payloads.append((codes, carrier)), metas.append(meta), owners.append(owner)
    gathered = tuple(torch.cat([p[i] for p in payloads], 0) for i in range(2))
    return owners, gathered, metas


@pytest.mark.parametrize(("experts", "world"), [(4, 4), (8, 4), (5, 4), (3, 4), (2, 4), (6, 1)])
def test_all_gather_payload_matches_whole_quantisation(experts, world):
    from gcore_lowp.fp8_tensor import Fp8TensorTrain, new_hook_stats
    say("fp8 all-gather payload", experts, world)
    n, k = 256, 384
    torch.manual_seed(experts * 16 + world)
    full = (torch.randn(experts, n, k) * 0.05)
    full[0, :128, :128] = 0                                  # a zero block: codes 0, scale byte 127
    module = types.SimpleNamespace(_fp8_all_gather_stats=new_hook_stats())
    owners, gathered, metas = _gather(full.cuda(), world, module)
    w, keep = owners[0].fsdp_post_all_gather(gathered, metas[0], torch.bfloat16)
    assert isinstance(w, Fp8TensorTrain) and tuple(w.shape) == (experts, n, k) and w.dtype == torch.bfloat16
    q_ref, s_ref = T.quant_fp8_e4m3_scale_e8m0(full, block_size=(128, 128))
    assert w._data.cpu().view(torch.uint8).equal(q_ref.view(torch.uint8))
    assert w._scale.cpu().view(torch.uint8).equal(s_ref.view(torch.uint8).reshape(experts, n // 128, k // 128))
    stats = module._fp8_all_gather_stats
    chunk = -(-experts // world)
    assert stats["pre_calls"] == world and stats["post_new_calls"] == 1
    assert stats["payload_dtype"] == "torch.uint8"
    assert stats["fp8_bytes"] == chunk * n * k and stats["fp8_bytes"] * 4 == stats["high_precision_bytes"]
    assert stats["scale_bytes"] == (chunk * n * k if experts % world else chunk * (n // 128) * (k // 128))
    assert stats["payload_bytes"] == stats["fp8_bytes"] + stats["scale_bytes"]
    # refresh of the same object on the next unshard
    assert owners[0].fsdp_post_all_gather(gathered, metas[0], torch.bfloat16, out=w) is None
    assert stats["post_reuse_calls"] == 1


def test_wrong_shard_shape_is_refused():
    from gcore_lowp.fp8_tensor import Fp8TensorAg, new_hook_stats
    say("fp8 all-gather wrong shard shape")
    module = types.SimpleNamespace(_fp8_all_gather_stats=new_hook_stats())
    owner = Fp8TensorAg(torch.zeros(2, 128, 128, device="cuda"))
    with pytest.raises(ValueError, match="local shape"):
        owner.fsdp_pre_all_gather(_Mesh(4, 3), torch.Size((5, 128, 128)), None, module, None)   # rank 3 holds 0 of 5
    with pytest.raises(AssertionError, match="not divisible"):
        Fp8TensorAg(torch.zeros(1, 128, 100, device="cuda")).fsdp_pre_all_gather(
            _Mesh(1, 0), torch.Size((1, 128, 100)), None, module, None)


def test_grouped_linear_takes_gathered_weight():
    from gcore_lowp import MyTeGroupedLinearFp8
    from gcore_lowp.fp8_tensor import new_hook_stats
    say("grouped linear on Fp8TensorTrain")
    experts, n, k = 4, 256, 512
    m_splits = [40, 0, 129, 64]
    torch.manual_seed(5)
    full = (torch.randn(experts, n, k) * 0.05).cuda()
    x = torch.randn(sum(m_splits), k, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    module = types.SimpleNamespace(_fp8_all_gather_stats=new_hook_stats())
    owners, gathered, metas = _gather(full, 2, module)
    w, _ = owners[0].fsdp_post_all_gather(gathered, metas[0], torch.bfloat16)
    lin = MyTeGroupedLinearFp8(experts)
    y = lin(x, w, m_splits)
    y_pair = lin(x.detach(), (w._data, w._scale), m_splits)
    y_hp = lin(x.detach(), full, m_splits)                   # quantised inside: the same codes and scales
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (sum(m_splits), n)
    assert torch.equal(y.detach(), y_pair) and torch.equal(y.detach(), y_hp)
    y.float().sum().backward()                               # dgrad flows through a pre-quantised weight
    assert x.grad is not None and torch.isfinite(x.grad).all()
    # reference bound for the forward against the fp32 product (tests/test_gfused/test_te_gemm_fp8.py:543-585)
    ref = torch.cat([x.detach().float()[sum(m_splits[:e]):sum(m_splits[:e + 1])] @ full[e].float().t()
                     for e in range(experts)])
    rel = (y.detach().float() - ref).norm() / ref.norm()
    assert rel < 0.05, rel
    # a weight whose scale grid does not match is refused before any launch
    from gcore_lowp.fp8_tensor import Fp8TensorTrain
    bad = Fp8TensorTrain(w._data, w._scale[:, :1], torch.bfloat16)
    with pytest.raises(AssertionError):
        lin(x.detach(), bad, m_splits)
