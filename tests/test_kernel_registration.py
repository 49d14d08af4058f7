"""The package's functions register with a registry of the reference's shape (gpatch_v4/kernel/registry.py:73-113:
register_kernel(name, fn, devices), ValueError on a second registration of a name for a device).  The registry used here
is a restatement of that contract, not the reference's module."""
import pytest


class Registry:
    def __init__(self):
        self.table = {}

    def register_kernel(self, name, fn, devices):
        assert devices is not None
        device_list = (devices,) if isinstance(devices, str) else tuple(devices)
        if not device_list:
            raise ValueError("At least one device must be specified")
        reg = self.table.setdefault(name, {})
        for d in device_list:
            if d in reg:
                raise ValueError(f"Kernel '{name}' for device '{d}' already registered")
            reg[d] = fn


def test_every_function_registers_under_the_reference_name():
    from gcore_lowp import kernel_registration as K
    r = Registry()
    names = K.register_lowp_kernels(r.register_kernel, devices=("cuda", "mi355x"))
    assert set(names) == set(K.lowp_kernels()) and len(names) >= 15
    for n in names:
        assert callable(r.table[n]["cuda"]) and r.table[n]["cuda"] is r.table[n]["mi355x"]
        assert r.table[n]["cuda"].__name__ in (n, "apply")          # the straight-through wrappers are autograd `apply`s
    with pytest.raises(ValueError):
        K.register_lowp_kernels(r.register_kernel, devices="cuda", only=["gemm_impl"])
    with pytest.raises(KeyError):
        K.register_lowp_kernels(Registry().register_kernel, devices="cuda", only=["linear_cross_entropy"])
    r2 = Registry()
    K.register_lowp_kernels(r2.register_kernel, devices="cuda", only=["gemm_impl", "act_quant"])
    assert set(r2.table) == {"gemm_impl", "act_quant"}
