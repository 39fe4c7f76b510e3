"""The reference's torch operator names over the HIP library: `load()` registers fbgemm::split_embedding_* for ROCm
tensors (see fbgemm_ops.cpp)."""
import os

_LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib", "librecsdk_torch_ops.so")
_loaded = False


def load():
    """Registers the operators; raises if the library has not been built (python -m recsdk_amd.torch_ops.build)."""
    global _loaded
    if _loaded:
        return _LIB
    if not os.path.isfile(_LIB):
        raise RuntimeError(f"{_LIB} is missing: run `python -m recsdk_amd.torch_ops.build`")
    import torch

    torch.ops.load_library(_LIB)
    _loaded = True
    return _LIB
