"""MI355X-native tensor-bundle path for execution-ucx (Axon).

Gathers N DLPack tensors into one contiguous HBM send buffer with a per-tensor
header and scatters a received buffer back, with hand-written HIP kernels for
gfx950 behind a C ABI (``include/axon_rocm.h``).  The HIP library is required:
nothing here computes on the CPU.
"""
from . import _capi, streams
from ._capi import (AxonRocmError, HeaderError, LengthError, MismatchError, NoDeviceError,
                    NoMessageError, NotImplementedForEager, UnsupportedMemoryError)
from .bundle import (BundlePlan, DLDataType, DLDevice, PackedBundle, TensorMeta, bundle_to_host, pack_bundle,
                     unpack_bundle)
from .device import (CpuDevice, CudaDevice, Device, DeviceType, RocmDevice, SyclDevice, auto_detect, cpu, cuda,
                     device_count, rocm, sycl)
from .dlpack import DLPackExport, TensorView, extract, extract_many
from .loopback import AmMessage, LoopbackAmContext
from .memory import DevicePool, PoolBuffer, RocmMemoryResourceManager
from .pipeline import StreamedTransfer
from .runtime import AxonRuntime
from .transfer import (classify_argument, flatten_arguments, recv_arguments, recv_tensors, regroup,
                       send_arguments, send_tensors)

__version__ = "0.1.0"


def library_path() -> str:
    return _capi.LIBRARY_PATH


def tune(**kwargs) -> None:
    """Set process-wide kernel tunables (read when a plan builds its tables)."""
    lib = _capi.load()
    for k, v in kwargs.items():
        _capi.check(lib.axr_tune_set(k.encode(), int(v)))
