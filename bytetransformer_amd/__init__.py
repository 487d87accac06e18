"""MI355X-native padding-free BERT encoder-layer forward.

The product is the native code under csrc/ (HIP kernels behind the C ABI of
include/bt_hip.h, the C++ BertTransformer API, and the PyTorch operator
torch.ops.ByteTransformer.BertTransformer).  This Python package only loads
those libraries and hands them device pointers; there is no Python or CPU
implementation to fall back to - a missing library raises.
"""
from ._lib import (LibraryMissing, host_lib, kernel_lib, lib_dir, load_th_op,  # noqa: F401
                   th_op_path)
from . import ops  # noqa: F401
from .encoder import BertEncoder, BertEncoderLayer, GraphedBertEncoder, encoder_forward  # noqa: F401
