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
    "mf_hogwild_inflight": (f32, [u32, i32, u32, u32, u32]),
    "mf_hogwild_inflight_capped": (f32, [u32, i32, u32, u32, u32, u32]),
    "mf_mascot_norm_blocks": (u32, [u32]),
    "mf_update_count": (u32, [u32, u32, u32]),
    "mf_auto_workers": (u32, [u32]),
    "mf_gpu_test_rmse": (C.c_int, [vp, u32, vp, vp, u32, u32, C.c_int, vp]),
    "mf_first_sample_rating_idx": (u32, [u32, u32, u32, u32, u32, f32]),
    "mf_lr_schedule": (f32, [f32, f32, u32]),
    "mf_window_start": (u32, [u64, u32, u32, u32, u32]),
    "mf_single_sgd_hogwild": (i32, [vp, u32, vp, vp, i32, u32, u32, u32, f32, f32, u64, u32, vp, vp]),
    "mf_mem_quant_sgd_hogwild": (i32, [vp, u32, vp, vp, i32, u32, u32, u32, f32, f32, u64, u32, vp, vp]),
    "mf_hot_row_table": (i32, [vp, u32, u32, f32, f32, f32, f32, vp, vp, vp, vp]),
    "mf_row_traffic_probe": (i32, [vp, u32, vp, vp, u32, u32, u64, vp, vp]),
    "mf_row_traffic_probe_sides": (i32, [vp, u32, vp, vp, u32, u32, u32, u64, vp, vp]),
    "mf_synth_baseline_config": (i32, [i32, vp]),
    "mf_generate_ratings": (i32, [vp, u64, u64, u64, vp, vp]),
    "mf_generate_ratings_host": (i32, [vp, u64, u64, u64, vp]),
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
    "mf_default_params": (None, [vp]),
    "mf_init_model": (i32, [vp, vp, u32, u32, u32, u64, i32]),
    "mf_train": (i32, [vp, vp, u32, u32, u32, vp, u32, vp, vp, vp]),
    "mf_group_end_indices": (u32, [vp, u32, u32, vp]),
    "mf_session_create": (i32, [vp, vp, u32, u32, u32, vp, u32, vp, vp, vp, vp]),
    "mf_session_epoch": (i32, [vp, vp, vp]),
    "mf_session_finish": (i32, [vp, vp, vp]),
    "mf_session_destroy": (None, [vp]),
    "mf_session_workers": (u32, [vp]),
    "mf_session_hot_rows": (i32, [vp, vp, vp, vp]),
    "mf_session_device_state": (i32, [vp, u32, vp, vp]),
    "mf_session_groups": (i32, [vp, i32, vp, vp, vp]),
    "mf_session_promote_groups": (i32, [vp, i32, vp, u32]),
    "mf_replicate_threshold": (f32, [f32, f32]),
    "mf_replica_step_scale": (f32, [f32, f32]),
    "mf_sort_by_count_workspace_bytes": (C.c_size_t, [u32]),
    "mf_sort_by_count_ws": (i32, [vp, vp, u32, vp, C.c_size_t, vp]),
    "mf_sort_by_count_static_max": (u32, []),
    "mf_sort_by_count_static": (i32, [vp, vp, u32, vp]),
    "mf_shuffle_ratings_workspace_bytes": (C.c_size_t, [u32]),
    "mf_shuffle_ratings_ws": (i32, [vp, vp, u32, u64, vp, C.c_size_t, vp]),
    "mf_synth_tables_bytes": (C.c_size_t, [vp]),
    "mf_synth_build_tables": (i32, [vp, u64, vp, C.c_size_t, vp]),
    "mf_generate_ratings_ws": (i32, [vp, u64, vp, u64, u64, vp, vp]),
    "mf_replica_sync_dense": (i32, [vp, u32, i32, vp, vp, u32, i32, vp]),
}
# the update launches with one more argument, const mf_hogwild_options*
for _name in ("mf_single_sgd_hogwild", "mf_mem_quant_sgd_hogwild", "mf_mpt_sgd_hogwild", "mf_muppet_sgd_hogwild", "mf_afp_sgd_hogwild", "mf_mascot_sgd_hogwild"):
    SIGNATURES[_name + "_opt"] = (i32, SIGNATURES[_name][1] + [vp])


f64 = C.c_double


class SynthConfig(C.Structure):
    """mf_synth_config of include/mascot_hip.h."""
    _fields_ = [("n_users", u32), ("n_items", u32), ("n_train", u64), ("n_test", u64), ("user_alpha", f32), ("item_alpha", f32),
                ("rank", u32), ("noise", f32), ("mean", f32), ("step", f32), ("lo", f32), ("hi", f32), ("bimodal", u32)]


class MfParams(C.Structure):
    """mf_params of include/mascot_hip.h."""
    _fields_ = [("lambda_", f32), ("learning_rate", f32), ("decay", f32), ("sample_ratio", f32), ("error_threshold", f32),
                ("interval", u32), ("user_group_num", u32), ("item_group_num", u32), ("k", u32), ("num_workers", u32),
                ("epoch", u32), ("thread_block_size", u32), ("version", u32), ("is_yahoo", u32), ("seed", u64),
                ("verbose", u32), ("cached_rows", u32), ("epoch_splits", u32), ("hot_row_inflight", f32), ("hot_row_inflight_early", f32), ("hot_row_early_epochs", u32),
                ("hot_rows", u32), ("replicate_inflight", f32), ("replica_merges", u32), ("replica_add_inflight", f32), ("replica_step_scale", f32), ("wg_counts_updates", u32), ("replica_step_epochs", u32),
                ("early_inflight", f32), ("early_inflight_epochs", u32), ("replicate_inflight_late", f32), ("replicate_late_from", u32)]


class HogwildOptions(C.Structure):
    """mf_hogwild_options of include/mascot_hip.h."""
    _fields_ = [("cached_rows", u32), ("launches", u32), ("user_keep", vp), ("item_keep", vp), ("user_slot", vp), ("item_slot", vp),
                ("user_slot_row", vp), ("item_slot_row", vp), ("user_replicas", vp), ("item_replicas", vp), ("user_slots", u32), ("item_slots", u32), ("replica_step_scale", f32), ("all_binary16", u32), ("resident_workers", u32)]


class MfReport(C.Structure):
    """mf_report of include/mascot_hip.h."""
    _fields_ = [("rmse_per_epoch", vp), ("lr_per_epoch", vp), ("sgd_ms_per_epoch", vp),
                ("user2sorted_idx", vp), ("item2sorted_idx", vp), ("user_group_end_idx", vp), ("item_group_end_idx", vp),
                ("user_group_prec_info", vp), ("item_group_prec_info", vp),
                ("user_group_num", u32), ("item_group_num", u32), ("test_reconst", vp),
                ("preprocess_ms", f64), ("switching_ms", f64), ("error_ms", f64), ("sgd_ms", f64), ("total_ms", f64),
                ("update_count", u32), ("muppet_final_bits", u32), ("muppet_bits_per_epoch", vp)]


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

    # ---- host-level helpers over numpy arrays ----------------------------------------------
    def synth_config(self, config):
        """The synthetic stand-in of BASELINE.json's configuration `config` (1..5)."""
        c = SynthConfig()
        self.mf_synth_baseline_config(config, C.addressof(c))
        return c

    def default_params(self, **kw):
        prm = MfParams()
        self.lib.mf_default_params(C.byref(prm))
        for key, val in kw.items():
            setattr(prm, "lambda_" if key == "lambda_" or key == "lam" else key, val)
        return prm

    def init_model(self, n_users, n_items, k, seed, half_rounded=False):
        p = np.empty((n_users, k), np.float32)
        q = np.empty((n_items, k), np.float32)
        self.call("mf_init_model", p.ctypes.data, q.ctypes.data, n_users, n_items, k, seed, int(half_rounded))
        return p, q

    def train(self, prm, R, n_users, n_items, test, p, q):
        """Runs mf_train; returns a dict with the per-epoch figures and (MASCOT) the sorted-space tables."""
        E = prm.epoch
        out = dict(rmse=np.zeros(E, np.float64), lr=np.zeros(E, np.float32), sgd_ms=np.zeros(E, np.float32),
                   user2sorted=np.zeros(n_users, np.uint32), item2sorted=np.zeros(n_items, np.uint32),
                   user_end=np.zeros(max(prm.user_group_num, 1), np.uint32), item_end=np.zeros(max(prm.item_group_num, 1), np.uint32),
                   user_prec=np.zeros(max(prm.user_group_num, 1), np.uint8), item_prec=np.zeros(max(prm.item_group_num, 1), np.uint8),
                   test_reconst=np.zeros(test.size, NODE), muppet_bits=np.zeros(E, np.uint8))
        rep = MfReport()
        rep.rmse_per_epoch = out["rmse"].ctypes.data
        rep.lr_per_epoch = out["lr"].ctypes.data
        rep.sgd_ms_per_epoch = out["sgd_ms"].ctypes.data
        rep.user2sorted_idx = out["user2sorted"].ctypes.data
        rep.item2sorted_idx = out["item2sorted"].ctypes.data
        rep.user_group_end_idx = out["user_end"].ctypes.data
        rep.item_group_end_idx = out["item_end"].ctypes.data
        rep.user_group_prec_info = out["user_prec"].ctypes.data
        rep.item_group_prec_info = out["item_prec"].ctypes.data
        rep.test_reconst = out["test_reconst"].ctypes.data
        rep.muppet_bits_per_epoch = out["muppet_bits"].ctypes.data
        R = np.ascontiguousarray(R)
        test = np.ascontiguousarray(test)
        self.call("mf_train", C.byref(prm), R.ctypes.data, R.size, n_users, n_items, test.ctypes.data, test.size,
                  p.ctypes.data, q.ctypes.data, C.byref(rep))
        out["report"] = rep
        out["user_end"] = out["user_end"][:rep.user_group_num]
        out["item_end"] = out["item_end"][:rep.item_group_num]
        out["user_prec"] = out["user_prec"][:rep.user_group_num]
        out["item_prec"] = out["item_prec"][:rep.item_group_num]
        return out


class Session:
    """mf_session_* over numpy arrays: the product's training driver, one epoch per call."""

    def __init__(self, h, prm, R, n_users, n_items, test, p, q):
        self.h, self.prm = h, prm
        self.R, self.test, self.p, self.q = np.ascontiguousarray(R), np.ascontiguousarray(test), p, q
        self.report = MfReport()
        self.ptr = vp()
        h.call("mf_session_create", C.byref(prm), self.R.ctypes.data, self.R.size, n_users, n_items, self.test.ctypes.data, self.test.size,
               p.ctypes.data, q.ctypes.data, C.byref(self.report), C.byref(self.ptr))
        self.epochs_done = 0

    def epoch(self):
        """Runs the next epoch; returns (test RMSE, milliseconds of its update launches)."""
        rmse, ms = C.c_double(0), C.c_float(0)
        self.h.call("mf_session_epoch", self.ptr, C.byref(rmse), C.byref(ms))
        self.epochs_done += 1
        return rmse.value, ms.value

    @property
    def workers(self):
        return self.h.lib.mf_session_workers(self.ptr)

    def hot_rows(self):
        u, v, f = u32(0), u32(0), f32(0)
        self.h.call("mf_session_hot_rows", self.ptr, C.byref(u), C.byref(v), C.byref(f))
        return u.value, v.value, f.value

    def device_state(self, epoch):
        """(device address of the session's ratings, address of the mf_hogwild_options of `epoch`)."""
        r, o = vp(), vp()
        self.h.call("mf_session_device_state", self.ptr, epoch, C.byref(r), C.byref(o))
        return r.value, o.value

    def groups(self, side):
        """(precision byte per group, training ratings per group) of side 0 (users) or 1 (items); empty without groups."""
        cap = max(1, self.prm.item_group_num if side else self.prm.user_group_num)
        n, prec, ratings = u32(0), np.zeros(cap, np.uint8), np.zeros(cap, np.uint64)
        self.h.call("mf_session_groups", self.ptr, side, C.byref(n), prec.ctypes.data, ratings.ctypes.data)
        return prec[:n.value].copy(), ratings[:n.value].copy()

    def promote_groups(self, side, mask):
        mask = np.ascontiguousarray(mask, np.uint8)
        self.h.call("mf_session_promote_groups", self.ptr, side, mask.ctypes.data, mask.size)

    def finish(self):
        self.h.call("mf_session_finish", self.ptr, self.p.ctypes.data, self.q.ctypes.data)
        return self.p, self.q

    def close(self):
        if self.ptr:
            self.h.lib.mf_session_destroy(self.ptr)
            self.ptr = vp()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


_handle = None


def load():
    global _handle
    if _handle is None:
        _handle = MascotHip()
    return _handle
