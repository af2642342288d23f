"""Python mirror of the operator / graph / optimizer layer (C ABI of include/rembrandt_operator.h).

Class and method names follow the reference's Rust API (src/operator/mod.rs, src/operator/loss.rs,
src/operator/worker.rs, src/opt/sgd/mod.rs); every method is one call into librembrandt_hip.so.
Failures raise `Panic`, mirroring the reference's panic-on-error behaviour.
"""
import ctypes as C

import numpy as np

from . import _lib

ACT = {"Identity": 0, "Rect": 1, "Logistic": 2, "Tanh": 3}
INIT = {"Disabled": 0, "Uniform": 1, "Normal": 2, "Xavier": 3, "KaimingFwd": 4}
POOL = {"Max": 0, "Average": 1}
MOMENTUM = {"Zero": 0, "Update": 1, "UpdateNesterov": 2, "Gradient": 3, "GradientNesterov": 4}
STEP = {"Constant": 0, "Anneal1": 1, "Anneal2": 2, "Anneal4": 3, "Decay": 4, "Inverse": 5}
BUF = {"out_act": 0, "out_delta": 1, "weights": 2, "bias": 3, "grad_weights": 4, "grad_bias": 5,
       "acc_grad_weights": 6, "acc_grad_bias": 7,
       # batch-normalised operators; "u<k>.<name>" addresses conv + batch-norm unit k (100*k + id)
       "bn_scale": 8, "bn_bias": 9, "bn_scale_grad": 10, "bn_bias_grad": 11, "bn_running_mean": 12, "bn_running_ivar": 13,
       "bn_cached_mean": 14, "bn_cached_ivar": 15, "acc_bn_scale_grad": 16, "acc_bn_bias_grad": 17, "pre_act": 18,
       "pre_delta": 19, "mid_act": 30, "mid_delta": 31}
BNORM_AVG = {"Cumulative": 0, "Exponential": 1}


def buf_id(which):
    """'weights' -> 2; 'u1.bn_scale' -> 108; integers pass through."""
    if isinstance(which, int):
        return which
    if which[0] == "u" and "." in which:
        unit, name = which.split(".", 1)
        return 100 * int(unit[1:]) + BUF[name]
    return BUF[which]


def _avg_args(mov_avg):
    """'Cumulative' | ('Exponential', ema_factor) -> (kind, ema_factor)"""
    if isinstance(mov_avg, str):
        return BNORM_AVG[mov_avg], 0.0
    return BNORM_AVG[mov_avg[0]], float(mov_avg[1])

_vp, _i32, _i64, _f, _int, _u64 = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_int, C.c_uint64
_P = C.POINTER

PROTOTYPES = {
    "rho_last_message": (C.c_char_p, []),
    "rho_config_new": (_int, [_P(_vp)]),
    "rho_config_free": (_int, [_vp]),
    "rho_config_data3d": (_int, [_vp, _i32, _i32, _i32, _int]),
    "rho_worker_graph_launches": (_int, [_vp, _P(_i64)]),
    "rho_config_conv2d": (_int, [_vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _int, _int, _f]),
    "rho_config_bnorm_conv2d": (_int, [_vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _int, C.c_double, C.c_double, _int, _int, _f]),
    "rho_config_stack_res_conv2d": (_int, [_vp, _i32, _i32, _i32, _int, C.c_double, C.c_double, _int, _int, _f]),
    "rho_config_proj_stack_res_conv2d": (_int, [_vp, _i32, _i32, _i32, _i32, _i32, _i32, _int, C.c_double, C.c_double, _int, _int,
                                                _f]),
    "rho_config_affine": (_int, [_vp, _i32, _i32, _int, _int, _f]),
    "rho_config_pool2d": (_int, [_vp, _i32, _i32, _i32, _i32, _i32, _i32, _int, _int]),
    "rho_config_softmax_kl_loss": (_int, [_vp, _i32]),
    "rho_config_data3d_crop": (_int, [_vp, _i32, _i32]),
    "rho_config_data3d_flip_x": (_int, [_vp]),
    "rho_config_data3d_subtract_mean": (_int, [_vp, _vp, _i64]),
    "rho_config_data3d_subtract_mean_file": (_int, [_vp, C.c_char_p]),
    "rho_config_data3d_pca_lighting_noise": (_int, [_vp, _vp, _vp, _f]),
    "rho_config_dropout": (_int, [_vp, _i32, _f]),
    "rho_config_local_res_norm": (_int, [_vp, _i32, _i32, _i32, _i32, _f, _f, _f]),
    "rho_config_params_len": (_int, [_vp, _P(_i64)]),
    "rho_config_from_model_file": (_int, [C.c_char_p, _P(_vp)]),
    "rho_worker_new": (_int, [_vp, _i32, _int, _u64, _u64, _int, _int, _P(_vp)]),
    "rho_worker_free": (_int, [_vp]),
    "rho_worker_set_overlap_backward": (_int, [_vp, _int]),
    "rho_worker_input_out_dims": (_int, [_vp, _P(_i32), _P(_i32), _P(_i32)]),
    "rho_worker_last_preproc_draws": (_int, [_vp, _P(_i32), _P(_i32), _P(_int), _vp, _i64, _P(_i64)]),
    "rho_worker_dropout_stream": (_int, [_vp, _i32, _P(_u64), _P(_u64), _P(_u64)]),
    "rho_worker_encode_params": (_int, [_vp, _vp, C.c_size_t, _P(C.c_size_t)]),
    "rho_worker_decode_params": (_int, [_vp, _vp, C.c_size_t, _P(C.c_size_t)]),
    "rho_worker_encode_state": (_int, [_vp, _vp, C.c_size_t, _P(C.c_size_t)]),
    "rho_worker_decode_state": (_int, [_vp, _vp, C.c_size_t, _P(C.c_size_t)]),
    "rho_worker_checkpoint_params": (_int, [_vp, _i64, C.c_char_p]),
    "rho_worker_checkpoint_state": (_int, [_vp, C.c_char_p]),
    "rho_worker_can_rollback": (_int, [_vp, C.c_char_p, _P(_i64)]),
    "rho_worker_rollback_params": (_int, [_vp, _i64, C.c_char_p]),
    "rho_worker_rollback_state": (_int, [_vp, C.c_char_p]),
    "rho_worker_hidden_count": (_int, [_vp, _P(_i32)]),
    "rho_worker_op_kind": (_int, [_vp, _i32, _P(C.c_char_p)]),
    "rho_worker_stream": (_vp, [_vp]),
    "rho_worker_sync": (_int, [_vp]),
    "rho_worker_init_params": (_int, [_vp, _u64, _u64]),
    "rho_worker_expose_host_frame_buf": (_int, [_vp, _i32, _P(_vp)]),
    "rho_worker_load_frames": (_int, [_vp, _i32]),
    "rho_worker_load_frames_f32": (_int, [_vp, _vp, _i32]),
    "rho_worker_stage_label": (_int, [_vp, _i32, _i32]),
    "rho_worker_load_labels": (_int, [_vp, _i32]),
    "rho_worker_stage_weight": (_int, [_vp, _i32, _f]),
    "rho_worker_load_weights": (_int, [_vp, _i32]),
    "rho_worker_store_loss": (_int, [_vp, _i32, _P(_f)]),
    "rho_worker_store_output_categories": (_int, [_vp, _i32]),
    "rho_worker_get_output_categories": (_int, [_vp, _i32, _vp]),
    "rho_worker_accuracy_count": (_int, [_vp, _i32, _P(_i32)]),
    "rho_worker_forward": (_int, [_vp, _i32, _int, _i64]),
    "rho_worker_backward": (_int, [_vp, _i32]),
    "rho_worker_regularize": (_int, [_vp, _f]),
    "rho_worker_accumulate_grads": (_int, [_vp, _f, _f]),
    "rho_worker_update_params": (_int, [_vp, _f]),
    "rho_worker_update_params2": (_int, [_vp, _f, _f]),
    "rho_worker_save_params": (_int, [_vp]),
    "rho_worker_restore_params": (_int, [_vp]),
    "rho_worker_reset": (_int, [_vp]),
    "rho_worker_backward_scaled": (_int, [_vp, _i32, _f]),
    "rho_worker_descend": (_int, [_vp, _f, _f, _int]),
    "rho_worker_reset_gradients": (_int, [_vp, _f]),
    "rho_worker_reset_loss": (_int, [_vp, _i32]),
    "rho_worker_accumulate_loss": (_int, [_vp, _i32]),
    "rho_worker_store_accumulated_loss": (_int, [_vp, _P(_f)]),
    "rho_sgd2_new": (_int, [_i32, _int, _P(_f), _P(_i64), _f, _f, _P(_vp)]),
    "rho_sgd2_free": (_int, [_vp]),
    "rho_sgd2_begin": (_int, [_vp, _vp]),
    "rho_sgd2_batch": (_int, [_vp, _vp, _i32]),
    "rho_sgd2_end_minibatch": (_int, [_vp, _vp, _int]),
    "rho_sgd2_iter_counter": (_int, [_vp, _P(_i64)]),
    "rho_worker_buffer": (_int, [_vp, _i32, _int, _P(_vp), _P(_i64)]),
    "rho_worker_read_buffer": (_int, [_vp, _i32, _int, _vp, _i64]),
    "rho_worker_write_buffer": (_int, [_vp, _i32, _int, _vp, _i64]),
    "rho_sgd_new": (_int, [_i32, _int, _P(_f), _P(_i64), _int, _f, _f, _P(_vp)]),
    "rho_sgd_free": (_int, [_vp]),
    "rho_sgd_begin": (_int, [_vp, _vp]),
    "rho_sgd_step": (_int, [_vp, _vp, _int]),
    "rho_sgd_iter_counter": (_int, [_vp, _P(_i64)]),
    "rho_sgd_set_iter_counter": (_int, [_vp, _i64]),
    "rho_sgd_step_size_at": (_int, [_vp, _i64, _P(_f)]),
    "rho_sgd_train_batch": (_int, [_vp, _vp, _i32, _int, _P(_f), _P(_i32)]),
    "rho_dataset_open": (_int, [C.c_char_p, C.c_char_p, C.c_char_p, _P(_vp)]),
    "rho_dataset_open_from_file": (_int, [C.c_char_p, C.c_char_p, _P(_vp)]),
    "rho_dataset_free": (_int, [_vp]),
    "rho_dataset_num_samples": (_int, [_vp, _P(_i64)]),
    "rho_dataset_frame_dims": (_int, [_vp, _P(_i32), _P(_i32), _P(_i32)]),
    "rho_dataset_get_sample": (_int, [_vp, _i64, _vp, _P(_i32)]),
    "rho_sgd_train": (_int, [_vp, _vp, _vp, _int, _u64, _vp, _vp, _vp]),
    "rho_sgd_validate": (_int, [_vp, _vp, _P(_f), _P(_f)]),
}


class TrainConfig(C.Structure):
    _fields_ = [("checkpoint_dir", C.c_char_p), ("resume_from", _i64), ("display_iters", _i64), ("checkpoint_iters", _i64),
                ("save_iters", _i64), ("valid_iters", _i64), ("checkpoint_discard", _int), ("max_iters", _i64), ("fused", _int)]


class TrainStats(C.Structure):
    _fields_ = [("iters", _i64), ("epochs", _i64), ("last_loss", _f), ("last_error", _f), ("valid_runs", _i64),
                ("valid_loss", _f), ("valid_error", _f), ("log_path", C.c_char * 512)]


ORDER = {"Sequential": 0, "RandomEpisode": 1, "CyclicEpisode": 2}

_bound = False


class Panic(RuntimeError):
    """The reference panics on every error of this layer; so does this mirror."""


def lib():
    global _bound
    handle = _lib.lib()
    if not _bound:
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _bound = True
    return handle


def _chk(code):
    if code != 0:
        msg = lib().rho_last_message()
        raise Panic(msg.decode() if msg else "error %d" % code)


def _init_args(init):
    """('Normal', std) | ('Uniform', half_range) | 'Xavier' | 'KaimingFwd' | 'Disabled'"""
    if isinstance(init, str):
        return INIT[init], 0.0
    return INIT[init[0]], float(init[1])


class SequentialOperatorConfig:
    """Fluent builder, src/operator/worker.rs:133-228.  Dimension triples are (width, height, channels)."""

    def __init__(self, handle=None):
        if handle is None:
            h = _vp()
            _chk(lib().rho_config_new(C.byref(h)))
            handle = h
        self._h = handle

    @classmethod
    def from_model_file(cls, path):
        h = _vp()
        _chk(lib().rho_config_from_model_file(str(path).encode(), C.byref(h)))
        return cls(h)

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                lib().rho_config_free(self._h)
            except TypeError:   # interpreter shutdown: module globals are already gone, the process frees the rest
                pass
            self._h = None

    def data3d(self, in_dims, normalize=False):
        _chk(lib().rho_config_data3d(self._h, in_dims[0], in_dims[1], in_dims[2], int(normalize)))
        return self

    def conv2d(self, in_dims, conv_size, conv_stride, conv_pad, out_channels, act_func="Rect", init_weights=("Normal", 0.01)):
        k, v = _init_args(init_weights)
        _chk(lib().rho_config_conv2d(self._h, in_dims[0], in_dims[1], in_dims[2], conv_size, conv_stride, conv_pad,
                                     out_channels, ACT[act_func], k, v))
        return self

    def bnorm_conv2d(self, in_dims, conv_size, conv_stride, conv_pad, out_channels, bnorm_mov_avg=("Exponential", 0.1),
                     bnorm_epsilon=1e-5, act_func="Rect", init_weights="KaimingFwd"):
        k, v = _init_args(init_weights)
        a, f = _avg_args(bnorm_mov_avg)
        _chk(lib().rho_config_bnorm_conv2d(self._h, in_dims[0], in_dims[1], in_dims[2], conv_size, conv_stride, conv_pad,
                                           out_channels, a, f, bnorm_epsilon, ACT[act_func], k, v))
        return self

    def stack_res_conv2d(self, in_dims, bnorm_mov_avg=("Exponential", 0.1), bnorm_epsilon=1e-5, act_func="Rect",
                         init_weights="KaimingFwd"):
        k, v = _init_args(init_weights)
        a, f = _avg_args(bnorm_mov_avg)
        _chk(lib().rho_config_stack_res_conv2d(self._h, in_dims[0], in_dims[1], in_dims[2], a, f, bnorm_epsilon, ACT[act_func],
                                               k, v))
        return self

    def proj_stack_res_conv2d(self, in_dims, out_dims, bnorm_mov_avg=("Exponential", 0.1), bnorm_epsilon=1e-5, act_func="Rect",
                              init_weights="KaimingFwd"):
        k, v = _init_args(init_weights)
        a, f = _avg_args(bnorm_mov_avg)
        _chk(lib().rho_config_proj_stack_res_conv2d(self._h, in_dims[0], in_dims[1], in_dims[2], out_dims[0], out_dims[1],
                                                    out_dims[2], a, f, bnorm_epsilon, ACT[act_func], k, v))
        return self

    def affine(self, in_channels, out_channels, act_func="Rect", init_weights=("Normal", 0.01)):
        k, v = _init_args(init_weights)
        _chk(lib().rho_config_affine(self._h, in_channels, out_channels, ACT[act_func], k, v))
        return self

    def pool2d(self, in_dims, pool_size, pool_stride, pool_pad, pool_op="Max", ceil_mode=False):
        _chk(lib().rho_config_pool2d(self._h, in_dims[0], in_dims[1], in_dims[2], pool_size, pool_stride, pool_pad,
                                     POOL[pool_op], int(ceil_mode)))
        return self

    # Data3dPreproc steps (src/operator/mod.rs:395-423), appended in call order
    def crop(self, crop_width, crop_height):
        _chk(lib().rho_config_data3d_crop(self._h, crop_width, crop_height))
        return self

    def flip_x(self):
        _chk(lib().rho_config_data3d_flip_x(self._h))
        return self

    def subtract_elemwise_mean(self, mean=None, mean_path=None):
        if mean_path is not None:
            _chk(lib().rho_config_data3d_subtract_mean_file(self._h, str(mean_path).encode()))
        else:
            mean = np.ascontiguousarray(mean, np.float32)
            _chk(lib().rho_config_data3d_subtract_mean(self._h, mean.ctypes.data, mean.size))
        return self

    def pca_lighting_noise(self, singular_vecs, singular_vals, std_dev):
        v = np.ascontiguousarray(singular_vecs, np.float32).reshape(9)
        l = np.ascontiguousarray(singular_vals, np.float32).reshape(3)
        _chk(lib().rho_config_data3d_pca_lighting_noise(self._h, v.ctypes.data, l.ctypes.data, std_dev))
        return self

    def dropout(self, channels, drop_ratio):
        _chk(lib().rho_config_dropout(self._h, channels, drop_ratio))
        return self

    def local_res_norm(self, in_dims, cross_size, scale, power, min_div):
        _chk(lib().rho_config_local_res_norm(self._h, in_dims[0], in_dims[1], in_dims[2], cross_size, scale, power, min_div))
        return self

    def softmax_kl_loss(self, num_categories):
        _chk(lib().rho_config_softmax_kl_loss(self._h, num_categories))
        return self

    def params_len(self):
        out = _i64()
        _chk(lib().rho_config_params_len(self._h, C.byref(out)))
        return out.value


class SequentialOperatorWorker:
    """src/operator/worker.rs:230-477 plus the Input/Loss operator calls the optimizer makes on it."""

    def __init__(self, config, batch_size, capability="Backward", shared_seed=(1, 2), device=0, fuse_epilogue=True,
                 bf16_forward=False, overlap_backward=True, graph_steps=False, fuse_tail=True, winograd=True):
        """graph_steps: SgdOpt.train_batch records a whole step into a HIP graph and replays it (launch-bound networks)."""
        h = _vp()
        flags = ((1 if fuse_epilogue else 0) | (2 if bf16_forward else 0) | (4 if overlap_backward else 0) | (8 if graph_steps else 0) |
                 (0 if fuse_tail else 16) | (0 if winograd else 32))
        _chk(lib().rho_worker_new(config._h, batch_size, 0 if capability == "Forward" else 1, shared_seed[0],
                                  shared_seed[1], device, flags, C.byref(h)))
        self._h = h
        self.batch_size = batch_size
        self.shared_seed = tuple(shared_seed)

    def close(self):
        if getattr(self, "_h", None):
            lib().rho_worker_free(self._h)
            self._h = None

    __del__ = close

    def graph_launches(self):
        n = _i64()
        _chk(lib().rho_worker_graph_launches(self._h, C.byref(n)))
        return n.value

    def set_overlap_backward(self, on):
        _chk(lib().rho_worker_set_overlap_backward(self._h, int(on)))

    def hidden_count(self):
        out = _i32()
        _chk(lib().rho_worker_hidden_count(self._h, C.byref(out)))
        return out.value

    def op_kind(self, idx):
        out = C.c_char_p()
        _chk(lib().rho_worker_op_kind(self._h, idx, C.byref(out)))
        return out.value.decode()

    def stream(self):
        return lib().rho_worker_stream(self._h)

    def sync(self):
        _chk(lib().rho_worker_sync(self._h))

    def init_params(self, shared_seed=None):
        s = shared_seed or self.shared_seed
        _chk(lib().rho_worker_init_params(self._h, s[0], s[1]))

    # InputOperator
    def load_frames_u8(self, frames):
        """frames: uint8 array [batch][c][h][w]; staged through expose_host_frame_buf then load_frames."""
        frames = np.ascontiguousarray(frames, np.uint8)
        n = frames.shape[0]
        flen = frames[0].size
        for b in range(n):
            p = _vp()
            _chk(lib().rho_worker_expose_host_frame_buf(self._h, b, C.byref(p)))
            C.memmove(p, frames[b].ctypes.data, flen)
        _chk(lib().rho_worker_load_frames(self._h, n))

    def reload_frames(self, batch_size):
        """Copies the frames already staged in the host frame buffer to the device again (load_frames)."""
        _chk(lib().rho_worker_load_frames(self._h, batch_size))

    def load_frames_f32(self, frames):
        frames = np.ascontiguousarray(frames, np.float32)
        _chk(lib().rho_worker_load_frames_f32(self._h, frames.ctypes.data, frames.shape[0]))

    def input_out_dims(self):
        w, h, c = _i32(), _i32(), _i32()
        _chk(lib().rho_worker_input_out_dims(self._h, C.byref(w), C.byref(h), C.byref(c)))
        return w.value, h.value, c.value

    def last_preproc_draws(self):
        """(crop_off_w, crop_off_h, flipped, alphas) of the input operator's last forward()."""
        ow, oh, fl, n = _i32(), _i32(), _int(), _i64()
        _chk(lib().rho_worker_last_preproc_draws(self._h, C.byref(ow), C.byref(oh), C.byref(fl), None, 0, C.byref(n)))
        alphas = np.zeros((n.value,), np.float32)
        if n.value:
            _chk(lib().rho_worker_last_preproc_draws(self._h, None, None, None, alphas.ctypes.data, n.value, None))
        return ow.value, oh.value, bool(fl.value), alphas

    def dropout_stream(self, idx):
        a, b, c = _u64(), _u64(), _u64()
        _chk(lib().rho_worker_dropout_stream(self._h, idx, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    # parameter / state blobs and checkpoints
    def _encode(self, fn):
        n = C.c_size_t()
        _chk(fn(self._h, None, 0, C.byref(n)))
        buf = (C.c_uint8 * n.value)()
        _chk(fn(self._h, buf, n.value, None))
        return bytes(buf)

    def encode_params(self):
        return self._encode(lib().rho_worker_encode_params)

    def encode_state(self):
        return self._encode(lib().rho_worker_encode_state)

    def decode_params(self, blob):
        n = C.c_size_t()
        _chk(lib().rho_worker_decode_params(self._h, C.c_char_p(blob), len(blob), C.byref(n)))
        return n.value

    def decode_state(self, blob):
        n = C.c_size_t()
        _chk(lib().rho_worker_decode_state(self._h, C.c_char_p(blob), len(blob), C.byref(n)))
        return n.value

    def checkpoint_params(self, t, prefix):
        _chk(lib().rho_worker_checkpoint_params(self._h, t, str(prefix).encode()))

    def checkpoint_state(self, prefix):
        _chk(lib().rho_worker_checkpoint_state(self._h, str(prefix).encode()))

    def can_rollback(self, prefix):
        t = _i64()
        _chk(lib().rho_worker_can_rollback(self._h, str(prefix).encode(), C.byref(t)))
        return None if t.value < 0 else t.value

    def rollback_params(self, prefix, t=None):
        _chk(lib().rho_worker_rollback_params(self._h, -1 if t is None else t, str(prefix).encode()))

    def rollback_state(self, prefix):
        _chk(lib().rho_worker_rollback_state(self._h, str(prefix).encode()))

    # LossOperator
    def stage_label(self, batch_idx, category):
        _chk(lib().rho_worker_stage_label(self._h, batch_idx, int(category)))

    def load_labels(self, batch_size):
        _chk(lib().rho_worker_load_labels(self._h, batch_size))

    def stage_weight(self, batch_idx, weight):
        _chk(lib().rho_worker_stage_weight(self._h, batch_idx, float(weight)))

    def load_weights(self, batch_size):
        _chk(lib().rho_worker_load_weights(self._h, batch_size))

    def stage_batch(self, labels, weight):
        for b, l in enumerate(labels):
            self.stage_label(b, int(l))
            self.stage_weight(b, weight)
        self.load_labels(len(labels))
        self.load_weights(len(labels))

    def store_loss(self, batch_size):
        out = _f()
        _chk(lib().rho_worker_store_loss(self._h, batch_size, C.byref(out)))
        return out.value

    def store_output_categories(self, batch_size):
        _chk(lib().rho_worker_store_output_categories(self._h, batch_size))

    def get_output_categories(self, batch_size):
        out = np.zeros((batch_size,), np.int32)
        _chk(lib().rho_worker_get_output_categories(self._h, batch_size, out.ctypes.data))
        return out

    def accuracy_count(self, batch_size):
        out = _i32()
        _chk(lib().rho_worker_accuracy_count(self._h, batch_size, C.byref(out)))
        return out.value

    # Operator
    def forward(self, batch_size, training=True, t=0):
        _chk(lib().rho_worker_forward(self._h, batch_size, int(training), t))

    def backward(self, batch_size):
        _chk(lib().rho_worker_backward(self._h, batch_size))

    def regularize(self, l2_reg_coef):
        _chk(lib().rho_worker_regularize(self._h, l2_reg_coef))

    def accumulate_grads(self, scale, momentum):
        _chk(lib().rho_worker_accumulate_grads(self._h, scale, momentum))

    def update_params(self, scale):
        _chk(lib().rho_worker_update_params(self._h, scale))

    def update_params2(self, grad_scale, update_scale):
        _chk(lib().rho_worker_update_params2(self._h, grad_scale, update_scale))

    def save_params(self):
        _chk(lib().rho_worker_save_params(self._h))

    def restore_params(self):
        _chk(lib().rho_worker_restore_params(self._h))

    # PipelineArchWorker::{backward, descend, reset_gradients} (src/arch_new.rs:534-551) and the second-generation loss
    # bookkeeping (src/layer_new.rs:2103-2134)
    def backward_scaled(self, batch_size, scale):
        _chk(lib().rho_worker_backward_scaled(self._h, batch_size, scale))

    def descend(self, scale, l2_reg_coef, fused=True):
        _chk(lib().rho_worker_descend(self._h, scale, l2_reg_coef, int(fused)))

    def reset_gradients(self, momentum):
        _chk(lib().rho_worker_reset_gradients(self._h, momentum))

    def reset_loss(self, batch_size):
        _chk(lib().rho_worker_reset_loss(self._h, batch_size))

    def accumulate_loss(self, batch_size):
        _chk(lib().rho_worker_accumulate_loss(self._h, batch_size))

    def store_accumulated_loss(self):
        out = _f()
        _chk(lib().rho_worker_store_accumulated_loss(self._h, C.byref(out)))
        return out.value

    def reset(self):
        _chk(lib().rho_worker_reset(self._h))

    # inspection
    def buffer_len(self, idx, which):
        p, n = _vp(), _i64()
        _chk(lib().rho_worker_buffer(self._h, idx, buf_id(which), C.byref(p), C.byref(n)))
        return n.value

    def device_ptr(self, idx, which):
        p, n = _vp(), _i64()
        _chk(lib().rho_worker_buffer(self._h, idx, buf_id(which), C.byref(p), C.byref(n)))
        return p.value, n.value

    def read(self, idx, which, count=None):
        n = self.buffer_len(idx, which) if count is None else count
        out = np.empty((n,), np.float32)
        _chk(lib().rho_worker_read_buffer(self._h, idx, buf_id(which), out.ctypes.data, n))
        return out

    def write(self, idx, which, values):
        values = np.ascontiguousarray(values, np.float32).ravel()
        _chk(lib().rho_worker_write_buffer(self._h, idx, buf_id(which), values.ctypes.data, values.size))


class DataSource:
    """MnistDataSource / Cifar10DataSource (src/data_new.rs:648-883), or an entry of a `.data` file."""

    def __init__(self, source=None, data_path=None, labels_path=None, data_file=None, key=None):
        h = _vp()
        if data_file is not None:
            _chk(lib().rho_dataset_open_from_file(str(data_file).encode(), key.encode(), C.byref(h)))
        else:
            _chk(lib().rho_dataset_open(source.encode(), str(data_path).encode(),
                                        str(labels_path).encode() if labels_path else None, C.byref(h)))
        self._h = h

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                lib().rho_dataset_free(self._h)
            except TypeError:   # interpreter shutdown: module globals are already gone, the process frees the rest
                pass
            self._h = None

    def num_samples(self):
        n = _i64()
        _chk(lib().rho_dataset_num_samples(self._h, C.byref(n)))
        return n.value

    def frame_dims(self):
        w, h, c = _i32(), _i32(), _i32()
        _chk(lib().rho_dataset_frame_dims(self._h, C.byref(w), C.byref(h), C.byref(c)))
        return w.value, h.value, c.value

    def get_sample(self, idx):
        w, h, c = self.frame_dims()
        frame = np.empty((c, h, w), np.uint8)
        cat = _i32()
        _chk(lib().rho_dataset_get_sample(self._h, idx, frame.ctypes.data, C.byref(cat)))
        return frame, cat.value


class SgdOptimization:
    """The per-minibatch block of the second-generation optimizer, src/opt_new.rs:279-325 (one worker): batches run
    forward -> backward(batch, 1.0) -> accumulate_loss with per-sample weights 1.0 (staged by the caller); a minibatch
    ends with descend(step_size.at_iter(t) / minibatch_size, l2) -> reset_gradients(momentum) -> t += 1."""

    def __init__(self, minibatch_size, step_size=0.01, momentum=0.9, l2_reg_coef=0.0):
        steps, iters = (_f * 5)(), (_i64 * 5)()
        steps[0] = step_size
        h = _vp()
        _chk(lib().rho_sgd2_new(minibatch_size, STEP["Constant"], steps, iters, momentum, l2_reg_coef, C.byref(h)))
        self._h = h

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                lib().rho_sgd2_free(self._h)
            except TypeError:
                pass
            self._h = None

    def begin(self, worker):
        _chk(lib().rho_sgd2_begin(self._h, worker._h))

    def batch(self, worker, batch_size):
        _chk(lib().rho_sgd2_batch(self._h, worker._h, batch_size))

    def end_minibatch(self, worker, fused=True):
        _chk(lib().rho_sgd2_end_minibatch(self._h, worker._h, int(fused)))

    def iter_counter(self):
        out = _i64()
        _chk(lib().rho_sgd2_iter_counter(self._h, C.byref(out)))
        return out.value


class SgdOpt:
    """The update block of SgdOpt::train, src/opt/sgd/new.rs:345-495 (one worker, no communication)."""

    def __init__(self, minibatch_size, step_size=0.01, momentum=("Update", 0.9), l2_reg_coef=0.0, schedule=None):
        steps = (_f * 5)()
        iters = (_i64 * 5)()
        kind = STEP["Constant"]
        if schedule is None:
            steps[0] = step_size
        else:
            kind = STEP[schedule["kind"]]
            for i, s in enumerate(schedule.get("steps", [])):
                steps[i] = s
            for i, it in enumerate(schedule.get("iters", [])):
                iters[i] = it
        mk, mu = (MOMENTUM[momentum], 0.0) if isinstance(momentum, str) else (MOMENTUM[momentum[0]], momentum[1])
        h = _vp()
        _chk(lib().rho_sgd_new(minibatch_size, kind, steps, iters, mk, mu, l2_reg_coef, C.byref(h)))
        self._h = h

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                lib().rho_sgd_free(self._h)
            except TypeError:   # interpreter shutdown: module globals are already gone, the process frees the rest
                pass
            self._h = None

    def begin(self, worker):
        _chk(lib().rho_sgd_begin(self._h, worker._h))

    def set_iter_counter(self, t):
        _chk(lib().rho_sgd_set_iter_counter(self._h, t))

    def train(self, worker, train_data, max_iters, valid_data=None, order="Sequential", order_seed=1, checkpoint_dir=None,
              resume_from=None, display_iters=0, checkpoint_iters=0, save_iters=0, valid_iters=0, checkpoint_discard=False,
              fused=True):
        """SgdOpt::train (src/opt/sgd/new.rs:209-639) for one worker, ended after max_iters minibatches."""
        cfg = TrainConfig(str(checkpoint_dir).encode() if checkpoint_dir else None, -1 if resume_from is None else resume_from,
                          display_iters, checkpoint_iters, save_iters, valid_iters, int(checkpoint_discard), max_iters, int(fused))
        st = TrainStats()
        _chk(lib().rho_sgd_train(self._h, worker._h, train_data._h, ORDER[order], order_seed,
                                 valid_data._h if valid_data is not None else None, C.byref(cfg), C.byref(st)))
        return {"iters": st.iters, "epochs": st.epochs, "last_loss": st.last_loss, "last_error": st.last_error,
                "valid_runs": st.valid_runs, "valid_loss": st.valid_loss, "valid_error": st.valid_error,
                "log_path": st.log_path.decode()}

    @staticmethod
    def validate(worker, valid_data):
        loss, acc = _f(), _f()
        _chk(lib().rho_sgd_validate(worker._h, valid_data._h, C.byref(loss), C.byref(acc)))
        return loss.value, acc.value

    def step(self, worker, fused=True):
        _chk(lib().rho_sgd_step(self._h, worker._h, int(fused)))

    def iter_counter(self):
        out = _i64()
        _chk(lib().rho_sgd_iter_counter(self._h, C.byref(out)))
        return out.value

    def step_size_at(self, t):
        out = _f()
        _chk(lib().rho_sgd_step_size_at(self._h, t, C.byref(out)))
        return out.value

    def train_batch(self, worker, batch_size, fused=True):
        loss, correct = _f(), _i32()
        _chk(lib().rho_sgd_train_batch(self._h, worker._h, batch_size, int(fused), C.byref(loss), C.byref(correct)))
        return loss.value, correct.value
