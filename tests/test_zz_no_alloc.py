"""The allocation-free variant of the inside forward+backward, ``pcfgnat_pcfg_loss_forward_backward_static``, called
through the C-ABI: its auxiliary table is a device array owned by the library instead of a buffer of the caller's.  The
kernels are those of ``pcfgnat_pcfg_loss_forward_backward``, so the results must be the same numbers: bit-equal where
one workgroup sweeps a sentence (graphs of up to 130 nodes), within the path's bar for fp32 (1e-4 of the gradient scale,
1e-5 relative on the log-likelihood) where the pipelined sweeps' exchange may resolve differently from run to run.

Two calls in a row share the array; the second is smaller, so it runs on whatever the first left behind.
"""
import pytest
import torch

from pcfg_nat_amd import _lib, harness, synth

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(B, L, T, seed, V=64):
    gen = torch.Generator().manual_seed(seed)
    src = torch.randint(max(2, L // 8), L // 4 + 1, (B,), generator=gen)
    src[0] = L // 4
    m = 4 * src
    n = (torch.round(1.1 * src.double()).long() + torch.randint(-2, 3, (B,), generator=gen)).clamp(min=2, max=T)
    n[0] = T
    batch = synth.training_batch(B, L, T, V, m, n, seed=seed)
    idx = batch["targets"].unsqueeze(1).expand(-1, L, -1)
    match = torch.log_softmax(batch["logits"], -1).gather(-1, idx)
    match = harness.eos_masked(match, batch["output_length"], batch["target_length"])
    go = torch.rand(B, generator=gen) + 0.5
    return [t.to(DEV).contiguous() for t in (go, match, batch["links"], batch["output_length"], batch["target_length"])]


def _run(lib, static, go, match, links, ol, tl):
    B, L, T = match.shape
    ml = links.size(2) - 1
    Mc = (L - 2) // (ml + 1) + 1
    S = torch.full((B, Mc, T + 2), float("nan"), device=DEV)
    mg = torch.full_like(match, float("nan"))
    lg = torch.full_like(links, float("nan"))
    st = torch.cuda.current_stream().cuda_stream
    if static:
        rc = lib.pcfgnat_pcfg_loss_forward_backward_static(go.data_ptr(), match.data_ptr(), links.data_ptr(), ol.data_ptr(),
                                                           tl.data_ptr(), S.data_ptr(), mg.data_ptr(), lg.data_ptr(), B, L, T, ml, st)
    else:
        aux = torch.empty((lib.pcfgnat_pcfg_aux_floats(B, L, T, ml),), dtype=torch.float32, device=DEV)
        rc = lib.pcfgnat_pcfg_loss_forward_backward(go.data_ptr(), match.data_ptr(), links.data_ptr(), ol.data_ptr(),
                                                    tl.data_ptr(), S.data_ptr(), aux.data_ptr(), mg.data_ptr(), lg.data_ptr(), B, L,
                                                    T, ml, st)
    _lib.check(rc, lib)
    torch.cuda.synchronize()
    return S[:, 0, 0].clone(), mg, lg


def _compare(static, plain, exact):
    for got, want in zip(static, plain):
        assert not torch.isnan(got).any()
        if exact:
            assert torch.equal(got, want)
        else:
            scale = want.abs().max()
            assert (got - want).abs().max() <= 1e-4 * scale
    if not exact:
        assert torch.allclose(static[0], plain[0], rtol=1e-5, atol=0)


def test_static_table_matches_caller_buffer_twice_in_a_row():
    lib = _lib.load()
    assert lib.pcfgnat_static_aux_floats() == 8 * 1024 * 1024
    # first call: long graphs (two pipelines of workgroups per sentence), 12 MiB of the 32 MiB table
    big = _inputs(4, 512, 140, seed=11)
    assert lib.pcfgnat_pcfg_aux_floats(4, 512, 140, 1) <= lib.pcfgnat_static_aux_floats()
    print("static inside forward+backward: B=4 L=512 T=140", flush=True)
    _compare(_run(lib, True, *big), _run(lib, False, *big), exact=False)
    # second call, smaller, on what the first left in the table: the training shape of the benchmark
    small = _inputs(40, 128, 32, seed=12)
    print("static inside forward+backward: B=40 L=128 T=32", flush=True)
    _compare(_run(lib, True, *small), _run(lib, False, *small), exact=True)
    # and the long shape once more after the short one
    print("static inside forward+backward: B=4 L=512 T=140 again", flush=True)
    _compare(_run(lib, True, *big), _run(lib, False, *big), exact=False)


def test_static_table_with_general_max_left():
    """The entry point also dispatches to the kernels for max_left != 1 (tables in the same static array): max_left = 2,
    two calls in a row, the second smaller; same kernels as the caller-buffer call, one workgroup per sentence: bit-equal."""
    lib = _lib.load()
    for B, L, T, ms, ns, seed in ((3, 32, 12, [32, 20, 8], [12, 9, 4], 21), (2, 20, 8, [20, 11], [8, 5], 22)):
        batch = synth.training_batch(B, L, T, 64, ms, ns, seed=seed, ml=2)
        idx = batch["targets"].unsqueeze(1).expand(-1, L, -1)
        match = harness.eos_masked(torch.log_softmax(batch["logits"], -1).gather(-1, idx), batch["output_length"],
                                   batch["target_length"])
        go = torch.linspace(0.5, 1.5, B)
        args = [t.to(DEV).contiguous() for t in (go, match, batch["links"], batch["output_length"], batch["target_length"])]
        assert args[2].size(2) == 3
        print("static inside forward+backward, max_left = 2: B=%d L=%d T=%d" % (B, L, T), flush=True)
        static, plain = _run(lib, True, *args), _run(lib, False, *args)
        assert torch.isfinite(plain[0]).all()
        _compare(static, plain, exact=True)


def test_static_table_rejects_what_does_not_fit():
    lib = _lib.load()
    B, L, T = 256, 512, 24
    assert lib.pcfgnat_pcfg_aux_floats(B, L, T, 1) > lib.pcfgnat_static_aux_floats()
    one = torch.zeros(1, device=DEV)
    ptr = one.data_ptr()  # never dereferenced: the size check comes first
    rc = lib.pcfgnat_pcfg_loss_forward_backward_static(ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, B, L, T, 1, None)
    assert rc == _lib.EINVAL
    assert b"static table" in lib.pcfgnat_last_error()
