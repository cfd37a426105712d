"""ctypes binding of libmascot_hip.so.  Device buffers are passed as integer addresses
(torch tensors' data_ptr()); nothing here computes anything on the host."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmascot_hip.so")
HEADER = os.path.join(os.path.dirname(HERE), "include", "mascot_hip.h")

NODE = np.dtype([("r", np.float32), ("u", np.uint32), ("i", np.uint32)], align=False)

u8, u16, u32, u64, i32, f32, vp = C.c_uint8, C.c_uint16, C.c_uint32, C.c_uint64, C.c_int, C.c_float, C.c_void_p

SIGNATURES = {
    "mf_version": (i32, []),
    "mf_last_error": (C.c_char_p, []),
    "mf_mascot_norm_blocks": (u32, [u32]),
    "mf_update_count": (u32, [u32, u32, u32]),
    "mf_first_sample_rating_idx": (u32, [u32, u32, u32, u32, u32, f32]),
    "mf_lr_schedule": (f32, [f32, f32, u32]),
    "mf_window_start": (u32, [u64, u32, u32, u32, u32]),
    "mf_single_sgd_hogwild": (i32, [vp, u32, vp, vp, i32, u32, u32, u32, f32, f32, u64, u32, vp, vp]),
    "mf_mpt_sgd_hogwild": (i32, [vp, u32, vp, vp, i32, u32, u32, u32, f32, u16, f32, u64, u32, vp, vp]),
    "mf_muppet_sgd_hogwild": (i32, [vp, u32, vp, vp, i32, u32, u32, u32, f32, f32, u32, vp, vp, u8, u8, u64, u32, vp, vp]),
    "mf_afp_sgd_hogwild": (i32, [vp, u32, vp, vp, i32, u32, u32, u32, f32, f32, i32, u64, u32, vp, vp]),
    "mf_mascot_sgd_hogwild": (i32, [vp, u32, vp, vp, i32, u32, u32, u32, f32, f32, vp, vp, vp, vp, vp, vp, vp, vp,
                                    u32, u32, u32, u64, u32, vp, vp]),
    "mf_transform_float2half": (i32, [vp, vp, u64, vp]),
    "mf_transform_half2float": (i32, [vp, vp, u64, vp]),
    "mf_cpyparams2grouped_params": (i32, [vp, vp, vp, vp, vp, i32, u32, u32, vp]),
    "mf_grouped_params2dense": (i32, [vp, vp, vp, vp, i32, u32, u32, vp]),
    "mf_group_error": (i32, [vp, vp, u32, vp, vp, vp, i32, u32, vp]),
    "mf_test_rmse": (i32, [vp, u32, vp, vp, i32, vp, vp]),
    "mf_test_rmse_grouped": (i32, [vp, u32, vp, vp, i32, vp, vp, vp, vp, u32, u32, vp, vp]),
    "mf_init_rand_feature": (i32, [vp, u64, u64, u64, vp]),
    "mf_init_idx_arr": (i32, [vp, u32, vp]),
    "mf_user_item_histogram": (i32, [vp, u32, vp, vp, vp]),
    "mf_sort_by_count": (i32, [vp, vp, u32, vp]),
    "mf_matrix_reconst_triplet": (i32, [vp, vp, vp, u32, vp]),
    "mf_shuffle_ratings": (i32, [vp, vp, u32, u64, vp]),
}


class MfError(RuntimeError):
    pass


class MascotHip:
    """Thin handle over the shared library; every method is the C function of the same name
    and raises MfError when it returns non-zero."""

    def __init__(self, path=LIB_PATH):
        if not os.path.exists(path):
            raise MfError("libmascot_hip.so is not built (%s); run `python -m icdm-2021_mascot_amd.build` or "
                          "__graft_entry__.build() first -- there is no fallback path" % path)
        # In a process that also uses PyTorch-ROCm for device memory there must be one HIP runtime:
        # torch bundles its own libamdhip64.so.7; importing it first makes the loader bind this
        # library's libamdhip64.so.7 dependency to the copy that is already loaded.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        self.lib = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.lib, name)
            fn.restype = res
            fn.argtypes = args

    def last_error(self):
        return self.lib.mf_last_error().decode()

    def call(self, name, *args):
        rc = getattr(self.lib, name)(*args)
        if rc != 0:
            raise MfError("%s failed with code %d: %s" % (name, rc, self.last_error()))
        return rc

    def __getattr__(self, name):
        if name.startswith("mf_"):
            fn = getattr(self.lib, name)
            if SIGNATURES[name][0] is i32 and name != "mf_version":
                return lambda *a: self.call(name, *a)
            return fn
        raise AttributeError(name)


_handle = None


def load():
    global _handle
    if _handle is None:
        _handle = MascotHip()
    return _handle
