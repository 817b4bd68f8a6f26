"""ctypes binding of libspio_hip.so (hipRTC + HIP module API).

Takes the place of the reference's spio/cuda package (driver.pyx,
nvrtc_ctypes.py).
"""

from .driver import (
    DeviceAttributes,
    Function,
    Module,
    Program,
    HipError,
    get_device_attributes,
    get_driver_version,
    get_runtime_version,
    get_hiprtc_version,
    init,
    is_initialized,
    library_path,
    loaded_runtime_libraries,
    synchronize,
    stream_synchronize,
    set_device,
    zero_fill_async,
    launch_sequence_timed,
)
