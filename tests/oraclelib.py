"""ctypes bindings of the CPU oracle (oracle/liboracle.so) and, where it was built, of the compiled
reference CPU backend (oracle/_ref/libodl_ref.so). Test infrastructure only: imported by tests, by the
smoke check and by the CPU-baseline leg of the benchmark, never by the shipped package."""
import atexit
import ctypes
import os
import shutil
import subprocess
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "liboracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libodl_ref.so")

_T = {"p": ctypes.c_void_p, "l": ctypes.c_int64, "i": ctypes.c_int, "f": ctypes.c_float}

# signature strings: p pointer, l int64, i int, f float; return type after '>' (i int, f float, l int64, v void)
_ORC_SIGS = {
    "orc_matmul": "ppplll>v",
    "orc_matmul_f64": "ppplll>v",
    "orc_im2col_f64": "plllliiiiiiip>i",
    "orc_col2im_f64": "plllliiiiiiip>i",
    "orc_conv2d_f64": "ppplllll" + "iiiiii" + "p>i",
    "orc_conv2d_backward_f64": "ppplllll" + "iiiiii" + "ppp>i",
    "orc_matmul_batched": "ppplllli>v",
    "orc_matmul_rows": "pppllll>v",
    "orc_transpose": "pplll>v",
    "orc_matmul_backward": "ppppplll>v",
    "orc_conv_outsize": "llll>l",
    "orc_im2col": "plllliiiiiiip>i",
    "orc_col2im": "plllliiiiiiip>i",
    "orc_conv2d": "ppplllll" + "iiiiii" + "p>i",
    "orc_conv2d_backward": "ppplllll" + "iiiiii" + "ppp>i",
    "orc_sum_axis": "plllp>v",
    "orc_sum_all": "pl>f",
    "orc_max_axis": "plllp>v",
    "orc_max_all": "pl>f",
    "orc_sum_to": "ppipip>i",
    "orc_broadcast_to": "ppipip>v",
    "orc_softmax": "plllp>v",
    "orc_gather": "ppillp>i",
    "orc_one_hot": "pillp>i",
    "orc_softmax_ce_loss": "ppillp>i",
    "orc_softmax_ce_grad": "ppillfp>i",
    "orc_max_pool2d": "plllliiiiiipp>i",
    "orc_max_pool2d_backward": "ppllll" + "iiiiii" + "p>i",
    "orc_argmax_rows": "pllp>v",
    "orc_accuracy": "ppll>f",
    "orc_binary": "iplplp>i",
    "orc_unary": "iplp>v",
    "orc_pow_scalar": "plfp>v",
    "orc_upsample_nearest": "p" + "llllll" + "ii" + "p>i",
    "orc_cat": "ppillp>i",
    "orc_yolo_detect_forward": "pppplp" + "lll" + "llll" + "f" + "ii" + "p>i",
    "orc_batch_norm_forward": "pppppif" + "lll" + "pppp>i",
    "orc_batch_norm_backward": "ppppf" + "lll" + "ppp>i",
    "orc_mlp_train_step": "ppillll" + "p" * 12 + "ifffff" + "pppppp>i",
    "orc_cnn_train_step": "ppillllll" + "p" * 8 + "f" + "p" + "pp" + "p" * 8 + "p>i",
}

_REF_SIGS = {
    "odl_ref_ping": ">i",
    "odl_ref_matmul": "ppplll>i",
    "odl_ref_matmul_batched": "pppllll" + "i>i",
    "odl_ref_matmul_fwd_bwd": "pppppplll>i",
    "odl_ref_transpose": "pppi>i",
    "odl_ref_im2col": "plllliiiiiiip>i",
    "odl_ref_col2im": "ppillll" + "iiiiiii" + "p>i",
    "odl_ref_conv2d": "ppplllll" + "iiiiii" + "p>i",
    "odl_ref_conv2d_backward": "pppplllll" + "iiiiii" + "ppp>i",
    "odl_ref_sum": "ppiiip>i",
    "odl_ref_max": "ppiip>i",
    "odl_ref_sum_to": "ppipip>i",
    "odl_ref_broadcast_to": "ppipip>i",
    "odl_ref_broadcast_to_backward": "ppipipp>i",
    "odl_ref_softmax": "ppiip>i",
    "odl_ref_gather": "ppillp>i",
    "odl_ref_one_hot": "pillp>i",
    "odl_ref_softmax_ce": "ppillpp>i",
    "odl_ref_max_pool2d": "plllliiiiiipp>i",
    "odl_ref_max_pool2d_backward": "ppllll" + "iiiiii" + "p>i",
    "odl_ref_accuracy": "ppllp>i",
    "odl_ref_binary": "ippippip>i",
    "odl_ref_unary": "iplp>i",
    "odl_ref_pow_scalar": "plfp>i",
    "odl_ref_activation": "iplp>i",
    "odl_ref_upsample": "p" + "llllll" + "ii" + "p>i",
    "odl_ref_cat": "ppillp>i",
    "odl_ref_pnnx_forward": "ppplllliplppp>i",
    "odl_ref_yolo_detect": "ppppp" + "ll" + "llll" + "f" + "ii" + "p>i",
    "odl_ref_batch_norm_forward": "pppppif" + "llll" + "pppp>i",
    "odl_ref_batch_norm_backward": "ppppppf" + "llll" + "ppp>i",
    "odl_ref_batch_norm_layer": "pllllifffi" + "ppp" + ">i",
    "odl_ref_save_mlp": "pp>i",
    "odl_ref_load_mlp": "pippp>i",
    "odl_ref_checkpoint_roundtrip": "ppiifffffppp>i",
    "odl_ref_mlp_train": "ppillll" + "pppp" + "ifffff" + "pppppp>i",
    "odl_ref_cnn_train": "ppillllll" + "p" * 8 + "f" + "p" + "p" * 8 + "p>i",
    "odl_ref_mlp_bench": "lllliipp>i",
    "odl_ref_cnn_bench": "liipp>i",
    "odl_ref_mlp_model_bench": "lllliiipp>i",
    "odl_ref_matmul_f64_fwd_bwd": "pppppplll>i",
    "odl_ref_conv2d_f64_fwd_bwd": "pppplllll" + "iiiiii" + "pppp>i",
    "odl_ref_softmax_f64_fwd_bwd": "pppiipp>i",
}


# entry points only the device build of the driver has (streams and recorded graphs do not exist in the reference)
_DEVICE_ONLY_SIGS = {
    "odl_host_mlp_train_graph": _REF_SIGS["odl_ref_mlp_train"],
    "odl_host_mlp_bench_graph": "lllliiipp>i",
    "odl_host_cnn_bench_graph": "liiipp>i",
    "odl_host_cnn_bn_bench": "liiipp>i",
    "odl_host_pnnx_forward_graph": _REF_SIGS["odl_ref_pnnx_forward"],
    "odl_host_pnnx_set_fusion": "i>i",
    "odl_host_pnnx_last_graph_nodes": "p>i",
    "odl_host_pnnx_last_host_ms": "p>i",
    "odl_host_upload_ordering": "lip>i",
    "odl_host_graph_abort_recovery": "pplllpp>i",
    "odl_host_pending_fill_semantics": "lp>i",
    "odl_host_paired_layers_match_separate_modules": "lp>i",
}


def _ret(c):
    return {"v": None, "i": ctypes.c_int, "f": ctypes.c_float, "l": ctypes.c_int64}[c]


class _Lib:
    def __init__(self, path, sigs):
        self._lib = ctypes.CDLL(path)
        self._keep = []
        for name, sig in sigs.items():
            args, ret = sig.split(">")
            fn = getattr(self._lib, name)
            fn.argtypes = [_T[c] for c in args]
            fn.restype = _ret(ret)

    def __getattr__(self, name):
        fn = getattr(self._lib, name)

        def call(*args):
            conv = []
            for a in args:
                if isinstance(a, np.ndarray):
                    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
                    conv.append(a.ctypes.data)
                elif a is None:
                    conv.append(None)
                else:
                    conv.append(a)
            return fn(*conv)

        return call


def build_oracle(force=False):
    """Compile the plain-C oracle (seconds). Building the checker is not using it."""
    src = os.path.join(ORACLE_DIR, "oracle.c")
    if force or not os.path.exists(ORACLE_SO) or os.path.getmtime(ORACLE_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "liboracle.so"], stdout=subprocess.DEVNULL)
    return ORACLE_SO


_oracle = None
_ref = None


def oracle():
    global _oracle
    if _oracle is None:
        build_oracle()
        _oracle = _Lib(ORACLE_SO, _ORC_SIGS)
    return _oracle


def have_ref():
    return os.path.exists(REF_SO)


REF_MANIFEST = os.path.join(ORACLE_DIR, "_ref", "MANIFEST")


def write_ref_manifest(names):
    """Called by the build once the reference-side binaries exist: the tests that run them then FAIL when one is
    missing; without a manifest (a tree that never had the reference beside it) they skip."""
    with open(REF_MANIFEST, "w") as f:
        f.write("\n".join(names) + "\n")


def ref_binary(name):
    """Path of oracle/_ref/<name>, or None when it is absent and nothing says that it was built. Raises when the build
    recorded it (oracle/_ref/MANIFEST, or ODL_REQUIRE_REF=1 in the environment) and the file is not there."""
    path = os.path.join(ORACLE_DIR, "_ref", name)
    if os.path.exists(path):
        return path
    promised = os.environ.get("ODL_REQUIRE_REF") == "1"
    if os.path.exists(REF_MANIFEST):
        with open(REF_MANIFEST) as f:
            promised = promised or name in f.read().split()
    if promised:
        raise FileNotFoundError("oracle/_ref/%s was built with this tree but is missing now" % name)
    return None


def ref():
    """The compiled reference CPU backend; only present where oracle/Makefile's `ref` target was built."""
    global _ref
    if _ref is None:
        lib = _Lib(REF_SO, _REF_SIGS)
        # the reference's logger creates originlog/origin.txt under the working directory the first time it is used:
        # let that happen in a scratch directory, not in the tree the tests run from
        here, scratch = os.getcwd(), tempfile.mkdtemp(prefix="odl_ref_log_")
        os.chdir(scratch)
        try:
            lib.odl_ref_ping()
        finally:
            os.chdir(here)
        atexit.register(shutil.rmtree, scratch, True)
        _ref = lib
    return _ref


DRIVER_DIR = os.path.join(ROOT, "tests", "lib")
HOST_DRIVER_SO = os.path.join(DRIVER_DIR, "libodl_host_driver.so")
HOST_CPU_DRIVER_SO = os.path.join(DRIVER_DIR, "libodl_hostcpu_driver.so")


def build_drivers():
    """tests/api_driver.cpp compiled against the C++ host layer (origindl_amd/lib/liborigin_host.so, which must exist)
    -> tests/lib/libodl_host_driver.so (tensors on the device) and tests/lib/libodl_hostcpu_driver.so (tensors left
    on the CPU). Plain g++, no device code; the benchmark's whole-step rows and the host-layer tests load them."""
    pkg = os.path.join(ROOT, "origindl_amd")
    os.makedirs(DRIVER_DIR, exist_ok=True)
    common = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-fPIC", "-Wall", "-Wno-unused-variable", "-shared",
              "-I" + os.path.join(pkg, "host", "include"), "-I" + os.path.join(ROOT, "include")]
    link = [os.path.join(ROOT, "tests", "api_driver.cpp"), "-L" + os.path.join(pkg, "lib"), "-lorigin_host", "-lodl_hip",
            "-Wl,-rpath,$ORIGIN/../../origindl_amd/lib"]
    for defs, out in ((["-DDRV_ON_DEVICE", "-DDRV_PREFIX=odl_host_"], HOST_DRIVER_SO),
                      (["-DDRV_PREFIX=odl_hostcpu_"], HOST_CPU_DRIVER_SO)):
        cmd = common + defs + ["-o", out] + link
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("driver build failed:\n" + " ".join(cmd) + "\n" + res.stdout)
    return HOST_DRIVER_SO, HOST_CPU_DRIVER_SO
_host = {}


def host_driver(cpu=False):
    """tests/api_driver.cpp compiled against this repository's C++ host layer (origindl_amd/host): the same calls
    the reference driver makes, running on the gfx950 backend (odl_host_*), or with tensors left on the CPU
    (odl_hostcpu_*, where every compute call must refuse)."""
    key = "hostcpu" if cpu else "host"
    if key not in _host:
        prefix = "odl_%s_" % key
        sigs = {k.replace("odl_ref_", prefix): v for k, v in _REF_SIGS.items()}
        if not cpu:
            sigs.update(_DEVICE_ONLY_SIGS)
        _host[key] = _Lib(HOST_CPU_DRIVER_SO if cpu else HOST_DRIVER_SO, sigs)
    return _host[key]


BIND_DRIVER_SO = os.path.join(ORACLE_DIR, "_ref", "libodl_bind_driver.so")
_bind = None


def binding_driver():
    """tests/api_driver.cpp compiled against the REFERENCE's own headers and linked to the reference's own Tensor /
    Operator / nn / optim objects, with the gfx950 binding (binding/src) underneath instead of the reference's device
    dispatcher and memory layer; tensors on the device (odl_bind_*). Built by `make -C oracle ref-binding`."""
    global _bind
    if _bind is None:
        sigs = {k.replace("odl_ref_", "odl_bind_"): v for k, v in _REF_SIGS.items()}
        lib = _Lib(BIND_DRIVER_SO, sigs)
        here, scratch = os.getcwd(), tempfile.mkdtemp(prefix="odl_bind_log_")  # (the reference's logger, as in ref())
        os.chdir(scratch)
        try:
            lib.odl_bind_ping()
        finally:
            os.chdir(here)
        atexit.register(shutil.rmtree, scratch, True)
        _bind = lib
    return _bind


def ptr_arr(arrays):
    """Host array of the data addresses of `arrays` (for entry points that take a pointer table)."""
    return np.asarray([a.ctypes.data for a in arrays], dtype=np.uint64)


def shape_arr(shape):
    return np.asarray(list(shape), dtype=np.int64)
