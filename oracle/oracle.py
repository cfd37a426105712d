"""ctypes binding of the CPU checker (test infrastructure only).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; nothing in the shipped package does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, "_build")

NODE = np.dtype([("r", np.float32), ("u", np.uint32), ("i", np.uint32)], align=False)
assert NODE.itemsize == 12


def build(force=False):
    """Compile liboracle.so / liboracle_soft.so with the Makefile next to this file."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


class AfpQ(C.Structure):
    _fields_ = [("r", C.c_int), ("n", C.c_int), ("itv", C.c_int), ("mov_avg_range", C.c_float)]


class SynthConfig(C.Structure):
    """orc_synth_config (= mf_synth_config of the library)."""
    _fields_ = [("n_users", C.c_uint32), ("n_items", C.c_uint32), ("n_train", C.c_uint64), ("n_test", C.c_uint64),
                ("user_alpha", C.c_float), ("item_alpha", C.c_float), ("rank", C.c_uint32), ("noise", C.c_float), ("mean", C.c_float),
                ("step", C.c_float), ("lo", C.c_float), ("hi", C.c_float), ("bimodal", C.c_uint32)]


class AfpState(C.Structure):
    _fields_ = [("user", AfpQ), ("item", AfpQ), ("backward", AfpQ),
                ("update_user_params_iter", C.c_int), ("update_item_params_iter", C.c_int),
                ("update_backward_iter", C.c_int), ("cur_iter", C.c_int),
                ("scaling_factor_p", C.c_float), ("scaling_factor_q", C.c_float),
                ("scaling_factor_back_prop", C.c_float)]


def _ptr(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


class Oracle:
    def __init__(self, soft=False):
        name = "liboracle_soft.so" if soft else "liboracle.so"
        # ORACLE_BUILD_DIR: a directory with another build of the checker (tests/test_oracle_mutants.py points the pin
        # tests at builds with one deliberate mistake each)
        path = os.path.join(os.environ.get("ORACLE_BUILD_DIR", _BUILD), name)
        if not os.path.exists(path):
            build()
        self.lib = lib = C.CDLL(path)
        u16, u32, u64, f32, f64, i32, vp = C.c_uint16, C.c_uint32, C.c_uint64, C.c_float, C.c_double, C.c_int, C.c_void_p
        sig = {
            "orc_float2half": (u16, [f32]), "orc_half2float": (f32, [u16]), "orc_double2half": (u16, [f64]),
            "orc_half_add": (u16, [u16, u16]), "orc_half_sub": (u16, [u16, u16]), "orc_half_mul": (u16, [u16, u16]),
            "orc_half_fma": (u16, [u16, u16, u16]),
            "orc_float2half_array": (None, [vp, vp, u64]), "orc_half2float_array": (None, [vp, vp, u64]),
            "orc_update_count": (u32, [u32, u32, u32]), "orc_sample_ratings_num": (u32, [u32, u32, f32]),
            "orc_is_error_check_epoch": (i32, [u32, u32, u32]),
            "orc_first_sample_rating_idx": (u32, [u32, u32, u32, u32, u32, f32]),
            "orc_lr_schedule": (f32, [f32, f32, u32]), "orc_window_start": (u32, [u64, u32, u32, u32, u32]),
            "orc_histogram": (None, [vp, u64, vp, u32, vp, u32]), "orc_sort_by_count": (None, [vp, u32, vp, vp]),
            "orc_grouping": (u32, [vp, u32, u32, vp]), "orc_reindex_tables": (None, [vp, u32, vp, u32, vp, vp, vp]),
            "orc_reindex": (None, [vp, u64, vp, vp]),
            "orc_group_lookup": (None, [u32, vp, u32, C.POINTER(u32), C.POINTER(u32)]),
            "orc_shuffle_keys": (None, [u64, u64, vp]), "orc_shuffle": (None, [u64, vp, vp, u64]),
            "orc_init_normal": (None, [u64, u64, vp, u64]),
            "orc_generate_ratings": (None, [vp, u64, u64, u64, vp]),
            "orc_sgd_update": (None, [i32, vp, vp, f32, f32, f32]),
            "orc_mem_quant_update": (None, [i32, vp, vp, f32, f32, f32]),
            "orc_mem_quant_epoch": (None, [i32, vp, u32, vp, vp, u32, u32, u32, f32, f32, u64, u32, vp, i32]),
            "orc_mpt_update": (None, [i32, vp, vp, f32, f32, u16, f32]),
            "orc_mascot_update": (None, [i32, vp, i32, vp, i32, f32, f32, f32, vp, vp, C.POINTER(f32), C.POINTER(f32)]),
            "orc_muppet_update": (None, [i32, vp, vp, f32, f32, f32, i32, i32, vp, C.POINTER(f32)]),
            "orc_afp_state_init": (None, [C.POINTER(AfpState)]),
            "orc_afp_update": (None, [i32, C.POINTER(AfpState), vp, vp, f32, f32, f32, i32, i32]),
            "orc_sgd_epoch": (None, [i32, vp, u32, vp, vp, u32, u32, u32, f32, f32, u64, u32, vp, i32]),
            "orc_mpt_epoch": (None, [i32, vp, u32, vp, vp, u32, u32, u32, f32, f32, f32, u64, u32, vp, i32]),
            "orc_muppet_epoch": (None, [i32, vp, u32, vp, vp, u32, u32, u32, f32, f32, u32, vp, vp, i32, i32, u64, u32, vp, i32]),
            "orc_afp_epoch": (None, [i32, vp, u32, vp, vp, u32, u32, u32, f32, f32, i32, u64, u32, vp, i32]),
            "orc_mascot_epoch": (None, [i32, vp, u32, vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, f32, f32, u32,
                                        vp, vp, vp, vp, u64, u32, vp, i32]),
            "orc_rmse": (f64, [i32, vp, u64, vp, vp]),
            "orc_rmse_grouped": (f64, [i32, vp, u64, vp, vp, vp, vp, vp, vp, u32, u32]),
            "orc_group_error": (None, [i32, u32, vp, vp, u32, vp, vp, vp]),
            "orc_muppet_ladder_step": (i32, [i32, i32, C.POINTER(i32), C.POINTER(i32), C.POINTER(f32), C.POINTER(i32), vp, vp]),
        }
        for n, (res, args) in sig.items():
            fn = getattr(lib, n)
            fn.restype = res
            fn.argtypes = args

    # ---- convenience wrappers over numpy arrays ------------------------------------
    def f2h(self, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        out = np.empty(a.shape, dtype=np.uint16)
        self.lib.orc_float2half_array(_ptr(a), _ptr(out), a.size)
        return out

    def h2f(self, a):
        a = np.ascontiguousarray(a, dtype=np.uint16)
        out = np.empty(a.shape, dtype=np.float32)
        self.lib.orc_half2float_array(_ptr(a), _ptr(out), a.size)
        return out

    def window_starts(self, seed, epoch, num_workers, update_count, nnz):
        out = np.empty((update_count, num_workers), dtype=np.uint32)
        for ite in range(update_count):
            for w in range(num_workers):
                out[ite, w] = self.lib.orc_window_start(seed, epoch, w, ite, nnz)
        return out

    def histogram(self, R, n_users, n_items):
        uc = np.empty(n_users, np.uint32)
        ic = np.empty(n_items, np.uint32)
        self.lib.orc_histogram(_ptr(R), R.size, _ptr(uc), n_users, _ptr(ic), n_items)
        return uc, ic

    def sort_by_count(self, cnt):
        cnt = np.ascontiguousarray(cnt, np.uint32)
        sc = np.empty_like(cnt)
        sid = np.empty_like(cnt)
        self.lib.orc_sort_by_count(_ptr(cnt), cnt.size, _ptr(sc), _ptr(sid))
        return sc, sid

    def grouping(self, sorted_cnt, requested):
        sorted_cnt = np.ascontiguousarray(sorted_cnt, np.uint32)
        end = np.empty(sorted_cnt.size, np.uint32)
        g = self.lib.orc_grouping(_ptr(sorted_cnt), sorted_cnt.size, requested, _ptr(end))
        return end[:g].copy()

    def reindex_tables(self, sorted_id, end_idx):
        n = sorted_id.size
        id2sorted = np.empty(n, np.uint32)
        id2group = np.empty(n, np.uint32)
        gsize = np.empty(end_idx.size, np.uint32)
        self.lib.orc_reindex_tables(_ptr(sorted_id), n, _ptr(end_idx), end_idx.size, _ptr(id2sorted), _ptr(id2group), _ptr(gsize))
        return id2sorted, id2group, gsize

    def group_lookup(self, idx, end_idx):
        g = C.c_uint32()
        row = C.c_uint32()
        self.lib.orc_group_lookup(int(idx), _ptr(end_idx), end_idx.size, C.byref(g), C.byref(row))
        return g.value, row.value

    def shuffle(self, seed, R):
        out = np.empty_like(R)
        self.lib.orc_shuffle(seed, _ptr(R), _ptr(out), R.size)
        return out

    def generate_ratings(self, cfg, seed, first, count):
        """Ratings [first, first + count) of the seeded synthetic stream; cfg: any ctypes structure laid out like SynthConfig."""
        out = np.empty(count, NODE)
        c = SynthConfig.from_buffer_copy(bytes(cfg))
        self.lib.orc_generate_ratings(C.addressof(c), seed, first, count, _ptr(out))
        return out

    def init_normal(self, seed, stream, n):
        out = np.empty(n, np.float32)
        self.lib.orc_init_normal(seed, stream, _ptr(out), n)
        return out

    def rmse(self, k, test, P, Q):
        return self.lib.orc_rmse(k, _ptr(test), test.size, _ptr(P), _ptr(Q))


class GroupedModel:
    """Host mirror of the grouped P/Q storage (one array per group) for the checker."""

    def __init__(self, k, end_idx, prec, arrays):
        self.k = k
        self.end_idx = np.ascontiguousarray(end_idx, np.uint32)
        self.prec = np.ascontiguousarray(prec, np.uint8)
        self.arrays = arrays            # list of np.uint16 / np.float32 arrays, [group_size*k]
        self.refresh()

    def refresh(self):
        self.ptrs = (C.c_void_p * len(self.arrays))(*[a.ctypes.data for a in self.arrays])

    @property
    def groups(self):
        return len(self.arrays)

    def group_sizes(self):
        e = self.end_idx.astype(np.int64)
        return np.diff(np.concatenate([[-1], e]))


_default = None


def get():
    global _default
    if _default is None:
        _default = Oracle()
    return _default
