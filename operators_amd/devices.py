"""Device numbers of the C ABI (include/infiniop.h `enum DeviceEnum`).

0..3 are the reference's (operatorspy/devices.py:1-5); DEVICE_AMD = 4 is the
one this library implements.
"""


class DeviceEnum:
    DEVICE_CPU = 0
    DEVICE_CUDA = 1
    DEVICE_BANG = 2
    DEVICE_ASCEND = 3
    DEVICE_AMD = 4
