"""Device flags of the script-form tests (reference operatorspy/tests/test_utils.py:5-24,
which has --cpu, --cuda, --bang and --ascend): this library carries one device,
so the one flag is --amd; torch calls that GPU "cuda" on a ROCm build."""
import argparse


def get_args():
    parser = argparse.ArgumentParser(description="Test Operator")
    parser.add_argument("--amd", action="store_true", help="Run AMD GPU (MI355X, gfx950) test")
    parser.add_argument("--device-id", type=int, default=0, help="GPU ordinal")
    return parser.parse_args()


def run(test_cases, test):
    """Run `test(lib, handle, "cuda", *case)` for every case on the device the
    flags select; without --amd nothing is selected and that is said."""
    from operators_amd import DeviceEnum, create_handle, destroy_handle, open_lib

    args = get_args()
    if not args.amd:
        print("no device selected: pass --amd")
        return 2
    import torch

    if not torch.cuda.is_available():
        raise SystemExit("--amd needs a GPU: the library has no CPU path")
    torch.cuda.set_device(args.device_id)
    lib = open_lib()
    handle = create_handle(lib, DeviceEnum.DEVICE_AMD, args.device_id)
    try:
        for case in test_cases:
            test(lib, handle, "cuda", *case)
    finally:
        destroy_handle(lib, handle)
    print("\033[92mTest passed!\033[0m")
    return 0


class described:
    """`with described(lib, t0, t1, ...) as cts:` - the tensors described to the library for the length of the block."""

    def __init__(self, lib, *tensors):
        self.lib, self.tensors = lib, tensors

    def __enter__(self):
        from operators_amd import to_tensor

        self.cts = [to_tensor(t, self.lib) for t in self.tensors]
        return self.cts

    def __exit__(self, *exc):
        from operators_amd import destroy_tensor

        for ct in self.cts:
            destroy_tensor(self.lib, ct)
        return False


def workspace_for(lib, query, desc, device):
    """(pointer or None, size) of the workspace `query(desc, &size)` asks for, and the tensor that owns it."""
    import ctypes

    from operators_amd import check_error, create_workspace

    size = ctypes.c_uint64(0)
    check_error(query(desc, ctypes.byref(size)))
    owner = create_workspace(size.value, device)
    return (owner.data_ptr() if owner is not None else None), size.value, owner


def laid_out(t, strides):
    """t's values in a tensor with the given element strides (None: as it is)."""
    from operators_amd import rearrange_tensor

    return t if strides is None else rearrange_tensor(t, strides)
