"""MI355X-native drop-in for the inference path of the `sparseconvnet` package.

Module classes keep the reference's names, constructor arguments and
`forward(input, increment=False)` signature (sparseconvnet/__init__.py of the reference);
everything below them runs in hand-written HIP kernels behind a C ABI.
"""
forward_pass_multiplyAdd_count = 0
forward_pass_hidden_states = 0

from .sparseConvNetTensor import SparseConvNetTensor  # noqa: E402
from .metadata import Metadata  # noqa: E402
from .sequential import Sequential, set_auto_compile, get_auto_compile  # noqa: E402
from .tables import JoinTable, AddTable, ConcatTable, Identity  # noqa: E402
from .ioLayers import InputLayer, OutputLayer  # noqa: E402
from .submanifoldConvolution import SubmanifoldConvolution, ValidConvolution  # noqa: E402
from .convolution import Convolution  # noqa: E402
from .deconvolution import Deconvolution  # noqa: E402
from .batchNormalization import BatchNormalization, BatchNormReLU, BatchNormLeakyReLU  # noqa: E402
from .networkInNetwork import NetworkInNetwork  # noqa: E402
from .pooling import MaxPooling, AveragePooling, UnPooling, SparseToDense  # noqa: E402
from .networkArchitectures import UNet  # noqa: E402
from .utils import (toLongTensor, optionalTensor, checkpoint_save, checkpoint_restore,  # noqa: E402
                    ssc_offset_permutation, convert_zmajor_state_dict)
from .compiled import compile, CompiledNet  # noqa: E402
from .incremental import set_mode as set_incremental_mode, get_mode as get_incremental_mode  # noqa: E402
