"""occamy_amd -- a gfx950 (MI355X) runtime for the operations Occamy's DNN
dialect lowers to, with Occamy's memory-pool planner and a DNN-program
compiler/executor standing where its DNN-to-LLVM lowering stands.

The compute path is the HIP library ``lib/libdnnrt.so`` (C ABI in
``include/dnnrt.h``); there is no CPU fallback: loading fails loudly if the
library has not been built.
"""
from . import _abi  # noqa: F401

__all__ = ["_abi"]
