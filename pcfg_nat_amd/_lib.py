"""ctypes binding of libpcfg_nat_hip.so (declared in include/pcfg_nat_hip.h).

Takes the place of the reference's JIT loader ``get_pcfg_kernel`` (fs_plugins/custom_ops/pcfg_loss.py:18-47): the
library is built ahead of time for gfx950 (``pcfg_nat_amd/csrc/Makefile``) and loaded once; a missing library or a
missing GPU is an error, never a silent fallback.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpcfg_nat_hip.so")
EXT_PATH = os.path.join(_HERE, "lib", "_pcfg_nat_torch.so")

OK, EINVAL, EUNSUPPORTED, EHIP = 0, 1, 2, 3
F16, F32, F64 = 0, 1, 2

_lib = None
_ext = None

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int

# name -> (restype, argtypes); mirrors include/pcfg_nat_hip.h and include/pcfg_nat_hip_testing.h one to one
SIGNATURES = {
    "pcfgnat_abi_version": (_int, []),
    "pcfgnat_last_error": (ctypes.c_char_p, []),
    "pcfgnat_logsoftmax_gather": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _int, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_logsoftmax_gather_eos": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _int, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_logsoftmax_gather_backward": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_logsoftmax_max": (_int, [_vp, _int, _vp, _vp, _i64, _i64, _i64, _vp]),
    "pcfgnat_logsoftmax_gather_lse": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_logsoftmax_gather_backward_lse": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_aux_floats": (ctypes.c_size_t, [_i64, _i64, _i64, _i64]),
    "pcfgnat_pipeline_config": (None, [_int, _int]),
    "pcfgnat_pipeline_outside_spin_limit": (None, [_int]),
    "pcfgnat_pipeline_redo_wait_limit": (None, [_int]),
    "pcfgnat_pipeline_redo_counts": (_int, [_vp, _vp, _vp, _int]),
    "pcfgnat_links_grad_range_limit": (None, [ctypes.c_float]),
    "pcfgnat_max_left3_tuned": (_int, [_int]),
    "pcfgnat_max_left3_counts": (_int, [_vp, _vp, _int]),
    "pcfgnat_max_left3_viterbi_counts": (_int, [_vp, _vp, _int]),
    "pcfgnat_max_left3_supported": (_int, [_i64, _i64]),
    "pcfgnat_pcfg_loss": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_loss_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_loss_forward_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_static_aux_floats": (ctypes.c_size_t, []),
    "pcfgnat_pcfg_loss_forward_backward_static": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_aux_elems_f64": (ctypes.c_size_t, [_i64, _i64, _i64, _i64]),
    "pcfgnat_pcfg_loss_f64": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_loss_backward_f64": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_best_tree_f64": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_viterbi_f64": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "pcfgnat_criterion_loss": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_criterion_step": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                      _i64, ctypes.c_float, _vp, _vp, _vp]),
    "pcfgnat_criterion_forward": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                         _i64, _i64, _vp]),
    "pcfgnat_criterion_backward": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_extract_links_pack": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_extract_links_forward": (_int, [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_extract_links_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                              _i64, _i64, _vp]),
    "pcfgnat_extract_links_unpack": (_int, [_vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_extract_links_fused_supported": (_int, [_int, _i64, _i64, _i64]),
    "pcfgnat_extract_links_fused_forward": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                                    _i64, _i64, _vp]),
    "pcfgnat_extract_links_fused_backward_supported": (_int, [_int, _i64, _i64, _i64]),
    "pcfgnat_extract_links_fused_backward_workspace_bytes": (ctypes.c_size_t, [_i64, _i64, _i64, _i64]),
    "pcfgnat_extract_links_fused_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                                     _i64, _i64, _vp]),
    "pcfgnat_glat_step": (_int, [_vp, _int, _vp, _vp, _vp, _int, _vp, _vp, _vp, ctypes.c_float, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                 _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_best_tree": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "pcfgnat_pcfg_viterbi": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "pcfgnat_viterbi_decoding": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "pcfgnat_viterbi_decode_workspace_bytes": (ctypes.c_size_t, [_i64, _i64, _i64]),
    "pcfgnat_viterbi_decode": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "pcfgnat_viterbi_decode_logits": (_int, [_vp, _int, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "pcfgnat_lookahead_decode": (_int, [_vp, _vp, ctypes.c_float, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "pcfgnat_viterbi_decoding_host": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64]),
}


def build(verbose=False):
    """Compile the library in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j4", "-B"]
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or out.returncode != 0:
        print(out.stdout)
    if out.returncode != 0:
        raise RuntimeError("building libpcfg_nat_hip.so failed")
    return LIB_PATH


def load():
    """Load the library (once) and attach the prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libpcfg_nat_hip.so is missing (%s): build it with `make -C pcfg_nat_amd/csrc` or "
            "`python -c 'import __graft_entry__ as g; g.build()'`; there is no CPU fallback" % LIB_PATH)
    import torch  # noqa: F401  (its HIP runtime must be the one this library binds to)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def load_ext():
    """The host side of the training operators as a torch extension (``csrc/torch_ext.cpp``: checks, allocation, autograd
    nodes and the C-ABI call in C++), built beside the library by the same Makefile.  Loaded once, after the library itself
    (the extension links to it).  Raises if it has not been built."""
    global _ext
    if _ext is not None:
        return _ext
    load()
    if not os.path.exists(EXT_PATH):
        raise RuntimeError("_pcfg_nat_torch.so is missing (%s): build it with `make -C pcfg_nat_amd/csrc`" % EXT_PATH)
    import importlib.util
    spec = importlib.util.spec_from_file_location("_pcfg_nat_torch", EXT_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    if mod.abi_version() != _lib.pcfgnat_abi_version():
        raise RuntimeError("_pcfg_nat_torch.so was built against another version of libpcfg_nat_hip.so: rebuild both")
    _ext = mod
    return mod


def check(rc, lib=None):
    if rc != OK:
        lib = lib or load()
        msg = lib.pcfgnat_last_error().decode("utf-8", "replace")
        raise RuntimeError(msg or ("libpcfg_nat_hip error code %d" % rc))
