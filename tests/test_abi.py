"""CPU-side checks of the boundary: the C-ABI library loads without a GPU, exports exactly what include/pcfg_nat_hip.h
declares, and its host-only entry point (the tree-to-sequence readout, a CPU function in the reference as well,
pcfg_loss.cpp:12-73) agrees with the oracle.  No GPU compute is called here."""
import os
import re

import numpy as np
import pytest
import torch

from oracle import oracle
from pcfg_nat_amd import _lib, custom_ops, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    names = set()
    for header in ("pcfg_nat_hip.h", "pcfg_nat_hip_testing.h"):  # the entry points, and the test hooks and counters
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(pcfgnat_\w+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), name
        assert name in _lib.SIGNATURES, "binding table lacks %s" % name
    assert sorted(_lib.SIGNATURES) == names
    assert lib.pcfgnat_abi_version() == 5
    assert lib.pcfgnat_pcfg_aux_floats(40, 128, 32, 1) == 40 * (6 * 64 * 34 + 6 * 36)
    # more than 128 main-chain nodes: six tables, the shifts (padded to 16 bytes), two link copies with rows of 64*ceil(Mc/64)
    assert lib.pcfgnat_pcfg_aux_floats(8, 512, 140, 1) == 8 * (6 * 256 * 142 + 144 + 4 * 256 * 256 + 4 * 256 * 142 + 16 * 144 + 4 + 4 * 256 * 142 + 16 * 144 + 2 * 144)
    assert lib.pcfgnat_pcfg_aux_floats(1, 282, 9, 1) == (6 * 141 * 11 + 13 + 3) // 4 * 4 + 4 * 141 * 192 + 4 * 192 * 11 + 12 * 13 + 4 + 4 * 192 * 11 + 12 * 13 + 2 * 14


def test_torch_extension_loads_without_gpu():
    """The host side of the training operators (a torch extension linked to the library) imports on a machine without a
    GPU, reports the library's ABI version and raises loud errors for CPU tensors before anything is enqueued."""
    ext = _lib.load_ext()
    assert ext.abi_version() == _lib.load().pcfgnat_abi_version()
    for name in ("cuda_pcfg_loss", "dag_logsoftmax_gather_inplace", "pcfg_criterion"):
        assert hasattr(ext, name)
    with pytest.raises(RuntimeError, match="GPU"):
        ext.cuda_pcfg_loss(torch.zeros(1, 8, 4), torch.zeros(1, 8, 2, 8), torch.tensor([8]), torch.tensor([4]))
    with pytest.raises(RuntimeError, match="GPU"):
        ext.dag_logsoftmax_gather_inplace(torch.zeros(1, 8, 16), torch.zeros(1, 8, 4, dtype=torch.int64))


def test_argument_errors_without_gpu():
    lib = _lib.load()
    rc = lib.pcfgnat_pcfg_loss(None, None, None, None, None, None, 2, 16, 4, 30, None)
    assert rc == _lib.EINVAL and b"max_left" in lib.pcfgnat_last_error()
    rc = lib.pcfgnat_logsoftmax_gather(None, 7, None, 0, 0, 0, None, 0, 1, 1, 8, 1, None)
    assert rc == _lib.EINVAL
    with pytest.raises(RuntimeError):
        _lib.check(rc)


def test_link_scorer_form_selection_without_gpu():
    """Which shapes the scorer with its products inside the kernels covers, what its backward needs as workspace, and its
    argument errors: host logic of the library, no GPU call."""
    lib = _lib.load()
    f16, f32, f64 = (custom_ops._DTYPE_CODE[t] for t in (torch.float16, torch.float32, torch.float64))
    for F in (16, 32, 64, 128):
        assert lib.pcfgnat_extract_links_fused_supported(f16, 128, 8, F) == 1
        assert lib.pcfgnat_extract_links_fused_backward_supported(f16, 128, 8, F) == (1 if F <= 64 else 0)
    for F in (8, 16, 32, 64):
        assert lib.pcfgnat_extract_links_fused_supported(f32, 128, 8, F) == 1
        assert lib.pcfgnat_extract_links_fused_backward_supported(f32, 128, 8, F) == 1
    for dtype, Lg, H, F in ((f16, 128, 8, 8), (f16, 128, 8, 48), (f32, 128, 8, 24), (f32, 128, 8, 128), (f64, 128, 8, 64),
                           (f16, 128, 3, 64), (f16, 1, 8, 64), (f16, 8193, 8, 64), (f32, 128, 16, 64)):
        assert lib.pcfgnat_extract_links_fused_supported(dtype, Lg, H, F) == 0, (dtype, Lg, H, F)
    assert lib.pcfgnat_extract_links_fused_backward_supported(f32, 128, 16, 64) == 1  # per-head tiles: no limit on heads x dimension
    B, Lg, H, F = 40, 128, 8, 64
    assert lib.pcfgnat_extract_links_fused_backward_workspace_bytes(B, Lg, H, F) == 4 * (2 * B * Lg * H + 3 * B * H * Lg + B * H * F)
    assert lib.pcfgnat_extract_links_fused_backward_workspace_bytes(B, 1, H, F) == 0
    rc = lib.pcfgnat_extract_links_fused_backward(None, None, None, None, None, None, None, f16, None, None, None, None, None, None,
                                                  2, 64, 8, 48, None)
    assert rc == _lib.EUNSUPPORTED and b"not built" in lib.pcfgnat_last_error()
    rc = lib.pcfgnat_extract_links_fused_backward(None, None, None, None, None, None, None, f16, None, None, None, None, None, None,
                                                  2, 64, 8, 64, None)
    assert rc == _lib.EINVAL and b"null pointer" in lib.pcfgnat_last_error()
    rc = lib.pcfgnat_extract_links_fused_forward(None, None, None, f32, None, None, 1, None, None, None, None, None, None, 0, 64, 8, 64, None)
    assert rc == _lib.OK  # an empty batch is no work


def test_ops_refuse_to_run_without_gpu():
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError, match="GPU"):
        custom_ops.cuda_pcfg_loss(torch.zeros(1, 8, 4), torch.zeros(1, 8, 2, 8), torch.tensor([8]), torch.tensor([4]))
    with pytest.raises(RuntimeError, match="GPU"):
        custom_ops.dag_logsoftmax_gather_inplace(torch.zeros(1, 8, 4), torch.zeros(1, 8, 2, dtype=torch.int64))


def test_host_readout_matches_oracle():
    ml, L = 1, 48
    m = torch.tensor([48, 32, 20, 8])
    gen = torch.Generator().manual_seed(21)
    links = synth.make_links(4, L, m, ml, gen)
    ob = torch.randn(4, L, generator=gen) - 1.0
    tokens = torch.randint(0, 6, (4, L), generator=gen)  # tiny vocabulary: repeats and pads (1) occur
    S, R, Lt, M = oracle.viterbi(ob.numpy(), links.numpy(), m.numpy(), dtype=np.float32)
    left_mask, _, _ = synth.support_masks(L, ml)
    for pred in ([5, 4, 3, 1], [11, 7, 2, 1], [2, 2, 2, 1]):
        pred_t = torch.tensor(pred)
        want = oracle.viterbi_decoding(pred_t.numpy(), m.numpy(), Lt, R, M, tokens.numpy(), left_mask.numpy(), 1)
        got = custom_ops.viterbi_decoding(pred_t, m, torch.from_numpy(Lt), torch.from_numpy(R), torch.from_numpy(M),
                                          tokens, left_mask, 1)
        assert got.dtype == torch.float32
        assert np.array_equal(got.numpy(), want)


def test_support_mask_conversion_is_kept_per_tensor_and_version():
    """The link scorer converts integer support masks to flag bytes once per tensor: the same tensor gives the kept copy,
    an in-place change or another tensor (also one with equal contents) gives a fresh one."""
    import torch
    from pcfg_nat_amd import custom_ops as ops
    m = torch.tensor([[0, 1], [2, 0]])
    a = ops._as_flag_mask(m)
    assert a.dtype == torch.bool and a.tolist() == [[False, True], [True, False]]
    assert ops._as_flag_mask(m) is a
    m[0, 0] = 5
    b = ops._as_flag_mask(m)
    assert b is not a and b.tolist() == [[True, True], [True, False]]
    other = m.clone()
    assert ops._as_flag_mask(other) is not b and ops._as_flag_mask(other).tolist() == b.tolist()
    flags = torch.tensor([True, False])
    assert ops._as_flag_mask(flags) is flags
