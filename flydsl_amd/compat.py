"""Optional import aliases for harness code written against the reference tree.

``install()`` registers, for every name that is not importable already, the modules the reference's preshuffle GEMM
harness imports (tests/kernels/test_preshuffle_gemm.py:21-39): ``flydsl.compiler`` / ``flydsl.expr`` /
``flydsl.runtime.device`` (the handful of names that harness uses), ``tests.utils``, ``tests.test_common`` and
``tests.kernels.utils.gemm_common_utils`` (host quantisers, layouts, timing, acceptance).  A real ``flydsl``
installation is never shadowed."""

from __future__ import annotations

import importlib.util
import sys
import types


def _module(name, **attrs):
    m = types.ModuleType(name)
    m.__dict__.update(attrs)
    return m


def get_rocm_arch() -> str:
    import torch

    if not torch.cuda.is_available():
        return "gfx950"
    return getattr(torch.cuda.get_device_properties(0), "gcnArchName", "gfx950").split(":")[0]


def install(force: bool = False) -> list:
    from . import compiler, expr, layout, quant, testing

    added = []

    def add(name, module):
        if not force:
            if name in sys.modules:
                return
            try:
                if importlib.util.find_spec(name) is not None:
                    return
            except (ImportError, ValueError, AttributeError):
                pass
        sys.modules[name] = module
        parent, _, child = name.rpartition(".")
        if parent and parent in sys.modules:
            setattr(sys.modules[parent], child, module)
        added.append(name)

    add("flydsl", _module("flydsl", __path__=[]))
    add("flydsl.compiler", compiler)
    add("flydsl.expr", expr)
    add("flydsl.runtime", _module("flydsl.runtime", __path__=[]))
    add("flydsl.runtime.device", _module("flydsl.runtime.device", get_rocm_arch=get_rocm_arch))
    add("tests", _module("tests", __path__=[]))
    add("tests.utils", _module("tests.utils", pertoken_quant=quant.pertoken_quant, shuffle_weight=layout.shuffle_weight,
                               get_dtype_max=quant.get_dtype_max))
    add("tests.test_common", _module("tests.test_common", run_perftest=testing.run_perftest, verify_output=testing.verify_output,
                                     checkAllclose=testing.checkAllclose))
    add("tests.kernels", _module("tests.kernels", __path__=[]))
    add("tests.kernels.utils", _module("tests.kernels.utils", __path__=[]))
    gcu = _module("tests.kernels.utils.gemm_common_utils", per_1x32_f4_quant=quant.per_1x32_f4_quant,
                  shuffle_weight_w4=layout.shuffle_weight_w4, shuffle_scale_w4=layout.shuffle_scale_w4,
                  mxfp4_to_f32=quant.mxfp4_to_f32, e8m0_to_f32=quant.e8m0_to_f32, f32_to_e8m0=quant.f32_to_e8m0,
                  f32_to_mxfp4=quant.f32_to_mxfp4, pack_uint4=quant.pack_uint4, fp4x2=quant.fp4x2, fp8_e8m0=quant.fp8_e8m0)
    add("tests.kernels.utils.gemm_common_utils", gcu)
    if "tests.kernels.utils" in sys.modules:
        setattr(sys.modules["tests.kernels.utils"], "gemm_common_utils", sys.modules.get("tests.kernels.utils.gemm_common_utils", gcu))
    return added
