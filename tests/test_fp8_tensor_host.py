"""Host behaviour of the FP8 weight wrappers (CPU, no kernel is launched): which ops keep the wrapper, what the
gathered-weight type refuses, flatten / unflatten, and how the post-all-gather hook takes the gathered bytes apart
(gpatch_v4/models/deepseek_v4/fp8_tensor.py:36-47,94-131,214-320)."""
import pytest
import torch

from gcore_lowp.fp8_tensor import Fp8TensorAg, Fp8TensorTrain, new_hook_stats


def test_ag_wrapper_dispatch():
    base = torch.arange(24, dtype=torch.float32).reshape(4, 3, 2)
    p = Fp8TensorAg(base.clone().requires_grad_(True))
    assert p.shape == base.shape and p.dtype == torch.float32 and p.requires_grad
    # structural and copy ops stay wrapped
    for out in (p.detach(), p.detach().view(4, 6), p.detach()[1:3], p.detach().clone(), torch.empty_like(p.detach()),
                p.detach().new_zeros(2, 2), p.detach().to(torch.float32, copy=True)):
        assert isinstance(out, Fp8TensorAg), type(out)
    parts = p.detach().split(2)
    assert all(isinstance(x, Fp8TensorAg) for x in parts) and parts[1]._tensor.equal(base[2:])
    # arithmetic computes on the backing tensor and leaves the wrapper
    s = p.detach() * 2
    assert not isinstance(s, Fp8TensorAg) and s.equal(base * 2)
    # copy_ updates the backing storage in place (reload after offload)
    q = Fp8TensorAg(torch.zeros_like(base))
    q.copy_(Fp8TensorAg(base))
    assert q._tensor.equal(base)
    names, ctx = p.__tensor_flatten__()
    assert names == ["_tensor"] and ctx is None
    r = Fp8TensorAg.__tensor_unflatten__({"_tensor": base}, None, None, None)
    assert isinstance(r, Fp8TensorAg) and r._tensor is base


def test_ag_wrapper_gradient_reaches_backing_dtype():
    w = Fp8TensorAg(torch.ones(2, 3))
    w.requires_grad_(True)
    (w * torch.arange(3.0)).sum().backward()
    assert w.grad is not None and w.grad.dtype == torch.float32
    assert torch.as_tensor(w.grad).reshape(2, 3).equal(torch.arange(3.0).expand(2, 3))


def test_train_wrapper_dispatch():
    data = torch.arange(2 * 128 * 128, dtype=torch.int64).remainder(251).to(torch.uint8).reshape(2, 128, 128)
    scale = torch.tensor([0.5, 2.0]).to(torch.float8_e8m0fnu).reshape(2, 1, 1)
    w = Fp8TensorTrain(data, scale, torch.bfloat16)
    assert w.dtype == torch.bfloat16 and w.shape == data.shape and not w.requires_grad
    d = w.detach()
    assert isinstance(d, Fp8TensorTrain) and d._scale is scale and d._data.equal(data)
    v = w.view(2, 128 * 128)
    assert isinstance(v, Fp8TensorTrain) and v.shape == (2, 128 * 128) and v._scale is scale
    assert isinstance(w[0:1], Fp8TensorTrain) and w[0:1]._data.equal(data[0:1])
    assert isinstance(w.clone(), Fp8TensorTrain)
    with pytest.raises(NotImplementedError):
        w + 1
    with pytest.raises(NotImplementedError):
        w.float()
    names, ctx = w.__tensor_flatten__()
    assert names == ["_data", "_scale"] and ctx == {"dtype": torch.bfloat16}
    r = Fp8TensorTrain.__tensor_unflatten__({"_data": data, "_scale": scale}, ctx, None, None)
    assert isinstance(r, Fp8TensorTrain) and r.dtype == torch.bfloat16 and r._data is data


@pytest.mark.parametrize(("experts", "world"), [(4, 4), (8, 4), (5, 4), (3, 4), (2, 4)])
def test_post_all_gather_reassembles_rank_major_bytes(experts, world):
    """Builds what the gather would deliver from known bytes and checks the hook's slicing, for even, uneven and
    empty shards (tests/test_gpatch_v4/test_fsdp2_fp8_all_gather.py:320-380 runs these splits on real ranks)."""
    n, k = 128, 256
    chunk = -(-experts // world)
    g = torch.Generator().manual_seed(experts * 10 + world)
    codes = torch.randint(0, 256, (world * chunk, n, k), dtype=torch.uint8, generator=g)
    scales = torch.randint(100, 140, (world * chunk, n // 128, k // 128), dtype=torch.uint8, generator=g)
    uneven = experts % world != 0
    per_rank = chunk * (n // 128) * (k // 128)
    if uneven:
        carrier = torch.zeros_like(codes)
        for r in range(world):
            carrier[r * chunk:(r + 1) * chunk].view(-1)[:per_rank] = scales[r * chunk:(r + 1) * chunk].reshape(-1)
    else:
        carrier = scales
    stats = new_hook_stats()
    meta = {"stats": stats, "is_uneven": uneven, "mesh_size": world, "orig_outer": experts, "chunk_outer": chunk,
            "scale_tail_shape": (n // 128, k // 128), "scale_numel_per_rank": per_rank}
    owner = Fp8TensorAg(torch.zeros(0, n, k))
    w, keep = owner.fsdp_post_all_gather((codes, carrier), meta, torch.bfloat16)
    assert isinstance(w, Fp8TensorTrain) and w.dtype == torch.bfloat16 and tuple(w.shape) == (experts, n, k)
    assert w._data.equal(codes[:experts])
    assert w._scale.dtype == torch.float8_e8m0fnu and w._scale.view(torch.uint8).equal(scales[:experts])
    assert keep[0] is codes and keep[1] is carrier
    assert stats["post_new_calls"] == 1 and stats["compute_dtype"] == "torch.bfloat16"
    # second unshard: the same object is refreshed in place
    codes2 = codes.flip(0).contiguous()
    assert owner.fsdp_post_all_gather((codes2, carrier), meta, torch.bfloat16, out=w) is None
    assert w._data.equal(codes2[:experts]) and stats["post_reuse_calls"] == 1
