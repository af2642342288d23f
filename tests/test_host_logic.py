"""CPU: host-side logic and the C-ABI surface (no kernel is launched here)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from rembrandt_amd import _lib, configs, operator, synth
from rembrandt_amd.operator import Panic, SequentialOperatorConfig, SgdOpt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_EXAMPLES = "/root/reference/examples"


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:rh|rho|rembrandt_kernel)_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    handle = C.CDLL(_lib.LIB_PATH)
    names = declared_symbols("rembrandt_hip.h") + declared_symbols("rembrandt_operator.h")
    assert len(names) > 80
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, missing
    # and the bindings cover the header
    bound = set(_lib.PROTOTYPES) | set(operator.PROTOTYPES)
    assert not [n for n in names if n not in bound], [n for n in names if n not in bound]
    assert b"gfx950" in _lib.lib().rh_version()


def _c_prototypes(header):
    """name -> argument count of every function include/<header> declares."""
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for name, args in re.findall(r"\b((?:rh|rembrandt_kernel)_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text):
        args = args.strip()
        out[name] = 0 if args in ("", "void") else len(args.split(","))
    return out


def _rust_prototypes(path):
    text = re.sub(r"//.*", "", open(path).read())
    block = text[text.index('extern "C" {'):]
    block = block[:block.index("\n}")]
    out = {}
    for name, args in re.findall(r"pub fn (\w+)\s*\(([^)]*)\)", block):
        out[name] = len([a for a in args.split(",") if a.strip()])
    return out


def test_rust_facade_binds_the_whole_kernel_abi():
    """rust/src/ffi.rs (source for the reference's toolchain; no rustc in this image) declares every function of
    include/rembrandt_hip.h with the same number of arguments and nothing else, every rh_* / rembrandt_kernel_*
    function the facade's sources call is declared there, and the configuration types carry the reference's fields."""
    header = _c_prototypes("rembrandt_hip.h")
    rust = _rust_prototypes(os.path.join(ROOT, "rust", "src", "ffi.rs"))
    assert len(header) > 80
    assert sorted(set(header) - set(rust)) == []
    assert sorted(set(rust) - set(header)) == []
    assert [(n, header[n], rust[n]) for n in header if header[n] != rust[n]] == []
    types = set(re.findall(r"pub (?:struct|enum|type) (\w+)", open(os.path.join(ROOT, "rust", "src", "ffi.rs")).read()))
    for src in ("operator.rs", "lib.rs"):
        text = re.sub(r"//.*", "", open(os.path.join(ROOT, "rust", "src", src)).read())
        used = set(re.findall(r"\b((?:rh|rembrandt_kernel)_[a-z0-9_]+)\b", text))
        assert sorted(used - set(rust) - types) == [], src
    op = open(os.path.join(ROOT, "rust", "src", "operator.rs")).read()
    # src/operator/mod.rs:1366-1389, 61-109; src/operator/worker.rs:52-76
    for needle in ("pub enum Conv2dFwdBackend", "pub enum Conv2dBwdBackend", "pub fwd_backend:", "pub bwd_backend:",
                   "fn decode_params(&mut self, _blob: &[u8]) -> usize", "fn encode_params(&mut self, _blob: &mut Vec<u8>)",
                   "fn decode_state(&mut self, _blob: &[u8]) -> usize", "fn encode_state(&mut self, _blob: &mut Vec<u8>)",
                   "pub trait InputOperator: Operator", "fn expose_host_frame_buf(&mut self, batch_idx: usize) -> &mut [u8]",
                   "fn load_frames(&mut self, batch_size: usize)", "fn input_operator(&mut self) -> &mut InputOperator",
                   "fn checkpoint_params(&mut self, _t: usize, _prefix: &Path)", "fn checkpoint_state(&mut self, _prefix: &Path)",
                   "fn can_rollback(&mut self, _prefix: &Path) -> Option<usize>",
                   "fn rollback_params(&mut self, _t: Option<usize>, _prefix: &Path)", "fn rollback_state(&mut self, _prefix: &Path)"):
        assert needle in op, needle
    # the folded paths the benchmark uses are reachable from the facade, and regularize launches nothing for l2 == 0
    for call in ("rh_conv2d_bwd_filter_bias(", "rh_conv2d_bwd_data_relu(", "rh_sgd_momentum_step_multi(", "rh_pool2d_bwd_relu("):
        assert call in op, call
    assert re.search(r"if l2_reg_coef > 0\.0 \{\s*axpy\(l2_reg_coef, &self\.weights", op)


def test_error_codes_without_gpu():
    lib = _lib.lib()
    g = _lib.ConvGeom(0, 3, 8, 8, 4, 3, 3, 1, 1)
    assert lib.rh_conv2d_fwd(C.byref(g), 1.0, 1, 1, 0.0, 1, None, None, 0, 0, None) == _lib.RH_E_INVALID
    g = _lib.ConvGeom(2, 3, 8, 8, 4, 3, 3, 1, 1)
    assert lib.rh_conv2d_fwd(C.byref(g), 1.0, None, None, 0.0, None, None, None, 0, 0, None) == _lib.RH_E_INVALID
    assert lib.rh_conv2d_fwd(C.byref(g), 1.0, 256, 256, 0.0, 256, None, None, 0, 0, None) == _lib.RH_E_WORKSPACE
    # bf16 operands exist for the forward pass with scalar-offset loaders only
    assert lib.rh_conv2d_fwd(C.byref(g), 1.0, 256, 256, 0.0, 256, None, 512, 1 << 20,
                             _lib.RH_MATH_BF16_MFMA_FP32ACC | _lib.RH_ALGO_GATHER, None) == _lib.RH_E_UNSUPPORTED
    assert lib.rh_conv2d_bwd_data(C.byref(g), 1.0, 256, 256, 0.0, 256, 512, 1 << 20, _lib.RH_MATH_BF16_MFMA_FP32ACC,
                                  None) == _lib.RH_E_UNSUPPORTED
    big = _lib.ConvGeom(4096, 512, 64, 64, 8, 3, 3, 1, 1)   # 32 GiB input: beyond the 2 GiB buffer-addressing limit
    assert lib.rh_conv2d_fwd(C.byref(big), 1.0, 256, 256, 0.0, 256, None, 512, 1 << 20, 0, None) == _lib.RH_E_LIMIT
    assert lib.rh_sgemm(0, 0, 4, 4, 4, 1.0, 256, 2, 256, 4, 0.0, 256, 4, None, 0, 0, None) == _lib.RH_E_INVALID  # lda < m
    p = _lib.PoolGeom(1, 1, 4, 4, 2, 2, 0, 7, 0)
    assert lib.rh_pool2d_fwd(C.byref(p), 256, 256, None, None) == _lib.RH_E_INVALID
    assert lib.rh_sgd_momentum_step(4, 256, 256, 256, -1.0, 0.1, 0.9, 1.0, 1, None) == _lib.RH_E_INVALID  # l2 >= 0
    assert lib.rh_error_string(_lib.RH_E_WORKSPACE) and lib.rh_error_string(0) == b"ok"


def test_workspace_and_shape_helpers():
    lib = _lib.lib()
    assert [lib.rh_conv2d_out_dim(n, k, s, p) for (n, k, s, p) in [(227, 11, 4, 0), (27, 5, 1, 2), (13, 3, 1, 1), (2, 5, 1, 0)]] == [55, 27, 13, 0]
    assert [lib.rh_pool2d_out_dim(n, 3, 2, 0, 0) for n in (55, 27, 13, 54)] == [27, 13, 6, 26]
    assert [lib.rh_pool2d_out_dim(n, 3, 2, 0, 1) for n in (54, 27, 13)] == [27, 13, 6]
    g = _lib.ConvGeom(256, 96, 27, 27, 256, 5, 5, 1, 2)
    fwd = lib.rh_conv2d_workspace_bytes(C.byref(g), _lib.RH_CONV_FWD)
    bwf = lib.rh_conv2d_workspace_bytes(C.byref(g), _lib.RH_CONV_BWD_FILTER)
    bwd = lib.rh_conv2d_workspace_bytes(C.byref(g), _lib.RH_CONV_BWD_DATA)
    assert fwd % 256 == 0 and bwf % 256 == 0 and bwd % 256 == 0
    assert fwd >= 2400 * 16 and bwd >= 6400 * 20 and bwf > fwd


def test_scratch_sized_once_covers_every_smaller_batch():
    """Operators allocate scratch once for batch_cap and then run any batch <= batch_cap (partial last batches,
    src/operator/mod.rs:1664,1722).  The need of a pass is not monotone in the batch, so the operators size with the
    *_upto functions: for every layer of the four networks and every batch up to the capacity the per-call need must
    fit, and the non-monotone case that made this necessary must still exist (else the *_upto functions are moot)."""
    lib = _lib.lib()
    non_monotone = 0
    for name, cap in (("lenet", 128), ("cifar10", 128), ("alexnet", 256), ("nin", 256)):
        for l in configs.NETWORKS[name]()[1]:
            if l[0] == "conv2d":
                (w, h, c), k, st, pad, out = l[1], l[2], l[3], l[4], l[5]
                g = _lib.ConvGeom(cap, c, h, w, out, k, k, st, pad)
                for ps in (_lib.RH_CONV_FWD, _lib.RH_CONV_BWD_FILTER, _lib.RH_CONV_BWD_DATA):
                    room = lib.rh_conv2d_workspace_bytes_upto(C.byref(g), ps)
                    at_cap = lib.rh_conv2d_workspace_bytes(C.byref(g), ps)
                    assert room >= at_cap and room % 256 == 0
                    for n in range(1, cap + 1):
                        gn = _lib.ConvGeom(n, c, h, w, out, k, k, st, pad)
                        need = lib.rh_conv2d_workspace_bytes(C.byref(gn), ps)
                        assert need <= room, (name, l, ps, n)
                        non_monotone += need > at_cap
                P = lib.rh_conv2d_out_dim(h, k, st, pad) * lib.rh_conv2d_out_dim(w, k, st, pad)
                room = lib.rh_conv2d_bwd_bias_workspace_bytes_upto(cap, out, P)
                assert all(lib.rh_conv2d_bwd_bias_workspace_bytes(n, out, P) <= room for n in range(1, cap + 1))
            elif l[0] == "affine":
                i, o = l[1], l[2]
                for (m, n, k, which) in ((o, cap, i, 1), (i, o, cap, 2), (i, cap, o, 1)):
                    room = lib.rh_sgemm_workspace_bytes_upto(m, n, k, which)
                    for b in range(1, cap + 1):
                        need = lib.rh_sgemm_workspace_bytes(m, b, k) if which == 1 else lib.rh_sgemm_workspace_bytes(m, n, b)
                        assert need <= room, (name, l, which, b)
    assert non_monotone > 0
    for (C_, plane) in ((64, 56 * 56), (512, 49)):
        room = lib.rh_bnorm_workspace_bytes_upto(256, C_, plane)
        assert all(lib.rh_bnorm_workspace_bytes(n, C_, plane) <= room for n in range(1, 257))


def test_rng_is_a_pure_function_of_seed_stream_index():
    a = synth.normal(5, 7, (1000,))
    assert np.array_equal(a, synth.normal(5, 7, (1000,)))
    assert np.array_equal(a[:100], synth.normal(5, 7, (100,)))            # element i independent of n
    assert not np.array_equal(a, synth.normal(5, 8, (1000,))) and not np.array_equal(a, synth.normal(6, 7, (1000,)))
    big = synth.normal(1, 2, (1 << 20,))                                   # threaded fill == serial fill
    assert np.array_equal(big[:1000], synth.normal(1, 2, (1000,)))
    assert abs(float(big.mean())) < 5e-3 and abs(float(big.std()) - 1.0) < 5e-3
    u = synth.uniform(3, 4, (1 << 18,), -2.0, 6.0)
    assert u.min() >= -2.0 and u.max() < 6.0 and abs(float(u.mean()) - 2.0) < 3e-2
    k = synth.integers(3, 5, (20000,), 10)
    assert k.min() == 0 and k.max() == 9 and np.bincount(k).min() > 1700
    # known answers of this generator (regression pin of the documented algorithm)
    golden = np.load(os.path.join(ROOT, "tests", "golden", "rng_kat.npz"))
    assert np.array_equal(synth.normal(0x5EED0004, 100, (16,)), golden["normal"])
    assert np.array_equal(synth.uniform(0x5EED0001, 100, (16,)), golden["uniform"])
    assert np.array_equal(synth.integers(0x5EED0004, 200, (16,), 1000), golden["integers"])


def test_network_definitions_match_the_reference_geometry():
    expect = {"lenet": (1256080, 64, 2.454272), "cifar10": (145578, 128, 8.858861568),
              "alexnet": (62378344, 256, 1689.780781056), "nin": (7595176, 128, 818.931105792)}
    for name, (params, batch, gflop) in expect.items():
        net = configs.NETWORKS[name]()
        assert configs.build_config(net).params_len() == params
        assert abs(configs.train_flops(net, batch) / 1e9 - gflop) < 1e-6
    dims, layers, ncat = configs.alexnet()
    convs = [l for l in layers if l[0] == "conv2d"]
    assert [l[1] for l in convs] == [(227, 227, 3), (27, 27, 96), (13, 13, 256), (13, 13, 384), (13, 13, 384)]
    assert [l[1] for l in layers if l[0] == "affine"] == [9216, 4096, 4096]
    assert [l[1][0] for l in configs.nin()[1] if l[0] == "pool2d"] == [54, 27, 13, 6]
    assert [l[1] for l in configs.cifar10()[1] if l[0] == "affine"] == [1024, 64]


def test_model_files_in_the_reference_grammar():
    ex = os.path.join(ROOT, "examples")
    assert SequentialOperatorConfig.from_model_file(os.path.join(ex, "lenet.model")).params_len() == 1256080
    assert SequentialOperatorConfig.from_model_file(os.path.join(ex, "alexnet.model")).params_len() == 62378344
    assert SequentialOperatorConfig.from_model_file(os.path.join(ex, "nin.model")).params_len() == 7595176
    with pytest.raises(Panic):
        SequentialOperatorConfig.from_model_file(os.path.join(ex, "does-not-exist.model"))


def test_model_parser_errors(tmp_path):
    def parse(text):
        p = tmp_path / "m.model"
        p.write_text(text)
        return SequentialOperatorConfig.from_model_file(p)
    data = '[[layer]]\nname = "data"\ntype = "data"\nraw_width = 8\nraw_height = 8\ncrop_width = 8\ncrop_height = 8\nchannels = 1\n'
    fc = '[[layer]]\nname = "fc"\ntype = "fully_conn"\nout_channels = 3\nact_func = "identity"\ninit_weights = { kind = "normal", mean = 0.0, std = 0.1 }\n'
    loss = '[[layer]]\nname = "loss"\ntype = "softmax_loss"\nnum_categories = 3\n'
    assert parse(data + fc + loss).params_len() == 64 * 3 + 3
    assert parse("# c\n" + data + "\n\n" + fc + "[opt]\nminibatch_size = 4 # ignored table\n" + loss).params_len() == 195
    lrn = '[[layer]]\nname = "n"\ntype = "local_res_norm"\ncross_size = 5\nscale = 0.0001\npower = 0.75\nmin_div = 2\n'
    drop = '[[layer]]\nname = "d"\ntype = "dropout"\ndrop_ratio = 0.5\n'
    assert parse(data + lrn + drop + fc + loss).params_len() == 195
    for bad in (data + fc,                                             # no loss layer
                fc + loss,                                             # no input for the first layer
                data + fc.replace('"identity"', '"relu"') + loss,      # act_func "relu" is not in the grammar (config.rs:123-129)
                data + fc.replace('type = "fully_conn"\n', "") + loss,  # 'layer' missing 'type' field
                data + fc + loss.replace("3", "4"),                    # input length != num_categories
                data + fc.replace("std = 0.1", "std = 1") + loss,      # as_float() rejects an integer
                data + fc.replace('kind = "normal"', 'kind = "xavier"') + loss,
                data + '[[layer]]\nname = "n"\ntype = "local_res_norm"\n' + fc + loss,   # missing cross_size
                data + '[[layer]]\nname = "d"\ntype = "dropout"\n' + fc + loss,          # missing drop_ratio
                data + "garbage line\n" + fc + loss):
        with pytest.raises(Panic):
            parse(bad)


@pytest.mark.skipif(not os.path.isdir(REF_EXAMPLES), reason="reference tree not mounted")
def test_reference_example_files():
    assert SequentialOperatorConfig.from_model_file(os.path.join(REF_EXAMPLES, "imagenet_nin.model")).params_len() == 7595176
    # 28 -> conv5 pad2 16ch -> pool2 -> 14x14x16 = 3136 -> fc100 -> fc10
    assert SequentialOperatorConfig.from_model_file(os.path.join(REF_EXAMPLES, "mnist_lenet.model")).params_len() == \
        (25 * 16 + 16) + (3136 * 100 + 100) + (100 * 10 + 10)
    with pytest.raises(Panic):   # not parseable by the reference's own parser either (pool tables lack 'type', act_func "relu")
        SequentialOperatorConfig.from_model_file(os.path.join(REF_EXAMPLES, "imagenet_alexnet.model"))


def test_resnet18_template_and_bnorm_builders():
    """The ResNet-18 template (src/templates/resnet.rs:367-520): operator sequence, extents, and the parameter count
    the reference's params_len formulas give (filter + 4 per batch-norm channel; conv.rs:97-103, 926-934, 2197-2207)."""
    dims, layers, ncat = configs.resnet18()
    assert dims == (224, 224, 3) and ncat == 1000
    assert [l[0] for l in layers] == ["bnorm_conv2d", "pool2d"] + ["stack_res_conv2d"] * 2 + \
        ["proj_stack_res_conv2d", "stack_res_conv2d"] * 3 + ["pool2d", "affine"]
    assert [l[2] for l in layers if l[0] == "proj_stack_res_conv2d"] == [(28, 28, 128), (14, 14, 256), (7, 7, 512)]
    assert layers[1][1] == (112, 112, 64) and layers[2][1] == (56, 56, 64) and layers[-1][1] == 512
    want = (7 * 7 * 3 * 64 + 4 * 64) + 512 * 1000 + 1000
    for c in (64, 128, 256, 512):
        want += (2 if c == 64 else 1) * 2 * (9 * c * c + 4 * c)                  # plain residual units
        if c > 64:
            want += 9 * (c // 2) * c + 9 * c * c + (c // 2) * c + 12 * c        # the projecting unit in front of them
    assert configs.build_config(configs.resnet18()).params_len() == want == 11699112
    with pytest.raises(Panic):   # the output extent must equal or halve the input extent
        SequentialOperatorConfig().proj_stack_res_conv2d((28, 28, 64), (9, 9, 128))
    with pytest.raises(Panic):
        SequentialOperatorConfig().bnorm_conv2d((8, 8, 3), 3, 1, 1, 4, bnorm_epsilon=0.0)
    with pytest.raises(KeyError):
        SequentialOperatorConfig().stack_res_conv2d((8, 8, 4), bnorm_mov_avg="Median")
    cfg = SequentialOperatorConfig().data3d((8, 8, 3)).bnorm_conv2d((8, 8, 3), 3, 2, 1, 4, "Cumulative").stack_res_conv2d((4, 4, 4))
    assert cfg.params_len() == (27 * 4 + 16) + 2 * (9 * 16 + 16)


def test_builder_preconditions():
    with pytest.raises(Panic):
        SequentialOperatorConfig().conv2d((8, 8, 1), 3, 0, 1, 4)       # stride 0
    with pytest.raises(Panic):
        SequentialOperatorConfig().affine(0, 4)
    with pytest.raises(KeyError):
        SequentialOperatorConfig().pool2d((8, 8, 1), 2, 2, 0, "Median")
    cfg = SequentialOperatorConfig().data3d((8, 8, 1)).conv2d((8, 8, 1), 3, 1, 1, 4).pool2d((8, 8, 4), 2, 2, 0).affine(64, 3).softmax_kl_loss(3)
    assert cfg.params_len() == (9 * 4 + 4) + (64 * 3 + 3)


def test_step_size_schedules():
    s = SgdOpt(64, schedule={"kind": "Anneal4", "steps": [1.0, 0.5, 0.25, 0.125, 0.0625], "iters": [0, 10, 20, 30, 40]})
    assert [s.step_size_at(t) for t in (0, 9, 10, 19, 20, 29, 30, 39, 40, 10 ** 6)] == [1.0, 1.0, 0.5, 0.5, 0.25, 0.25, 0.125, 0.125, 0.0625, 0.0625]
    s = SgdOpt(64, schedule={"kind": "Anneal1", "steps": [0.1, 0.01], "iters": [0, 5]})
    assert [round(s.step_size_at(t), 6) for t in (4, 5)] == [0.1, 0.01]
    s = SgdOpt(64, schedule={"kind": "Inverse", "steps": [0.1, 0.01]})
    assert abs(s.step_size_at(100) - 0.1 / (1 + 0.1 * 0.01 * 100)) < 1e-7
    assert SgdOpt(64, 0.25).step_size_at(12345) == 0.25
    with pytest.raises(Panic):
        SgdOpt(64, schedule={"kind": "Decay", "steps": [0.1]}).step_size_at(0)   # unimplemented!() in the reference too
    assert SgdOpt(64, 0.1).iter_counter() == 0


def _write_idx(path, arr):
    import struct
    arr = np.ascontiguousarray(arr, np.uint8)
    with open(path, "wb") as f:
        f.write(struct.pack(">I", 0x0800 | arr.ndim))
        for d in arr.shape:
            f.write(struct.pack(">I", d))
        f.write(arr.tobytes())


def test_mnist_and_cifar_sources(tmp_path):
    """idx / CIFAR-binary readers (src/data_new.rs:648-883): header parsing, frame dims, sample access, the
    `.data` file route, and the malformed-file panics."""
    from rembrandt_amd.operator import DataSource
    rng = np.random.default_rng(3)
    imgs = rng.integers(0, 256, (11, 6, 9), dtype=np.uint8)       # 11 frames of 6 rows x 9 columns
    labels = rng.integers(0, 10, (11,), dtype=np.uint8)
    _write_idx(tmp_path / "img.idx", imgs)
    _write_idx(tmp_path / "lab.idx", labels)
    ds = DataSource("mnist", tmp_path / "img.idx", tmp_path / "lab.idx")
    assert ds.num_samples() == 11 and ds.frame_dims() == (9, 6, 1)
    for i in (0, 5, 10):
        frame, cat = ds.get_sample(i)
        assert np.array_equal(frame[0], imgs[i]) and cat == labels[i]
    with pytest.raises(Panic):
        ds.get_sample(11)
    recs = np.zeros((7, 3073), np.uint8)
    recs[:, 0] = np.arange(7)
    recs[:, 1:] = rng.integers(0, 256, (7, 3072), dtype=np.uint8)
    (tmp_path / "c.bin").write_bytes(recs.tobytes())
    cs = DataSource("cifar10", tmp_path / "c.bin")
    assert cs.num_samples() == 7 and cs.frame_dims() == (32, 32, 3)
    frame, cat = cs.get_sample(4)
    assert cat == 4 and np.array_equal(frame.ravel(), recs[4, 1:])
    (tmp_path / "d.data").write_text('[dataset.train]\nsource = "mnist"\ndata_path = "%s"\nlabels_path = "%s"\n'
                                     '[dataset.valid]\nsource = "cifar10"\ndata_path = "%s"\n'
                                     % (tmp_path / "img.idx", tmp_path / "lab.idx", tmp_path / "c.bin"))
    assert DataSource(data_file=tmp_path / "d.data", key="train").num_samples() == 11
    assert DataSource(data_file=tmp_path / "d.data", key="valid").frame_dims() == (32, 32, 3)
    # malformed inputs
    (tmp_path / "short.bin").write_bytes(b"\0" * 3000)
    _write_idx(tmp_path / "lab_short.idx", labels[:5])
    (tmp_path / "badmagic.idx").write_bytes(b"\0\0\x0d\x03" + b"\0" * 12)
    (tmp_path / "trunc.idx").write_bytes((tmp_path / "img.idx").read_bytes()[:-3])
    for args in (("cifar10", tmp_path / "short.bin", None), ("mnist", tmp_path / "img.idx", None),
                 ("mnist", tmp_path / "img.idx", tmp_path / "lab_short.idx"), ("mnist", tmp_path / "badmagic.idx", tmp_path / "lab.idx"),
                 ("mnist", tmp_path / "trunc.idx", tmp_path / "lab.idx"), ("mnist", tmp_path / "nope.idx", tmp_path / "lab.idx"),
                 ("episodb", tmp_path / "img.idx", None)):
        with pytest.raises(Panic):
            DataSource(*args)
    with pytest.raises(Panic):
        DataSource(data_file=tmp_path / "d.data", key="test")
