"""GPU: the two measurement entry points (tri_diag_issue_probe, tri_diag_power_probe) run, refuse what they do not
support, and report times that make sense (an MFMA of 32 matrix-pipe cycles cannot take fewer than 32 ticks)."""
import ctypes

import pytest
import torch

from trinity_amd import ext

pytestmark = pytest.mark.gpu


def test_issue_probe_counts_what_an_mfma_takes(dev):
    ticks, ns = ext.issue_probe(True, 0, 0, 2, iters=1024, workgroups=8)
    # two waves per SIMD, one MFMA per group: a SIMD needs at least 32 cycles per MFMA, i.e. 64 ticks per group
    assert 60.0 < ticks < 200.0 and ns > 0.0
    t8, _ = ext.issue_probe(True, 8, 0, 2, iters=1024, workgroups=8)
    t16, _ = ext.issue_probe(True, 16, 0, 2, iters=1024, workgroups=8)
    assert t16 > t8 > ticks * 0.95, "more vector instructions per group cannot take less time"
    # four waves per SIMD: the SIMD's time per group of one wave stays at an MFMA's 32 cycles or above
    t4, _ = ext.issue_probe(True, 0, 0, 4, iters=1024, workgroups=8)
    assert t4 / 4 > 31.0


def test_power_probe_runs_every_supported_mix(dev):
    base = None
    for nl, ng, nv, nt in ((0, 0, 0, 0), (2, 0, 0, 0), (4, 0, 0, 0), (0, 0, 4, 0), (0, 0, 4, 1), (0, 2, 0, 0),
                           (1, 2, 0, 0), (2, 2, 3, 1), (1, 2, 3, 1), (0, 4, 0, 0)):
        for rnd in (1, 0):
            ticks, ns, ghz = ext.power_probe(nl, ng, nv, nt, rnd, iters=2048, workgroups=8)
            assert ticks >= 31.0, "a SIMD cannot start two MFMAs within 32 cycles"
            assert ns > 0.0 and 0.5 < ghz < 3.5
            if (nl, ng, nv, nt, rnd) == (0, 0, 0, 0, 1):
                base = ticks
    assert base < 40.0, "MFMAs alone issue back to back"


def test_probes_refuse_unsupported_counts(dev):
    UNSUPPORTED, SHAPE = -6, -3   # TRI_ERR_UNSUPPORTED, TRI_ERR_SHAPE
    buf = torch.zeros(8 * 16 + 16, dtype=torch.uint8, device=dev)
    i32 = ctypes.c_int32
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    power = lambda nl, ng, nv, nt, iters: ext._call(
        "tri_diag_power_probe", [i32(nl), i32(ng), i32(nv), i32(nt), i32(1), i32(iters), i32(8), buf, st], True)
    # three LDS reads per two groups, five vector instructions, three loads per eight groups: not in the lists
    assert power(3, 0, 0, 0, 64) == UNSUPPORTED
    assert power(0, 0, 5, 0, 64) == UNSUPPORTED
    assert power(0, 3, 0, 0, 64) == UNSUPPORTED
    assert power(0, 0, 0, 0, 12) == SHAPE   # the loop count must be a multiple of eight
    issue = ext._call("tri_diag_issue_probe", [i32(1), i32(3), i32(0), i32(2), i32(64), i32(8), buf, st], True)
    assert issue == UNSUPPORTED
    small = torch.zeros(64, dtype=torch.uint8, device=dev)   # too small for eight workgroups
    assert ext._call("tri_diag_power_probe", [i32(0), i32(0), i32(0), i32(0), i32(1), i32(64), i32(8), small, st], True) == SHAPE
    torch.cuda.synchronize()
