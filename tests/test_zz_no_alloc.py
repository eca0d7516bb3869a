"""eet_mmha_decode_static (the entry point that allocates nothing: split partials in a static
device array) against eet_mmha_decode with a caller workspace, through the C ABI.  Same kernels,
same launch shapes, so the outputs must be bit-identical; two calls in a row share the array, the
second with a smaller input."""
import numpy as np
import pytest
import torch

from eet_amd._lib import check, lib

from gpu_util import mmha, stream

pytestmark = pytest.mark.gpu


def static_call(q, k, v, kc, vc, step, pad=None, alibi=None, rope_row=None):
    B, H, T, dh = kc.shape
    ctx = torch.empty(B, H * dh, dtype=torch.float16, device=kc.device)
    check(lib().eet_mmha_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, kc.data_ptr(), vc.data_ptr(),
                                       ctx.data_ptr(), alibi.data_ptr() if alibi is not None else None,
                                       pad.data_ptr() if pad is not None else None, B, H, dh, step, T,
                                       rope_row.data_ptr() if rope_row is not None else None, stream()),
          "eet_mmha_decode_static")
    return ctx


def case(gpu, seed, B, H, dh, step, alibi=False, pad=None):
    g = torch.Generator().manual_seed(seed)
    cap = step + 3
    kc = torch.randn(B, H, cap, dh, generator=g).half().to(gpu)
    vc = torch.randn(B, H, cap, dh, generator=g).half().to(gpu)
    q, k, v = [torch.randn(B, H, dh, generator=g).half().to(gpu) for _ in range(3)]
    bias = (torch.rand(H, step, generator=g) * 4).half().to(gpu) if alibi else None
    padt = torch.tensor(pad, dtype=torch.long, device=gpu) if pad is not None else None
    return q, k, v, kc, vc, bias, padt


def test_static_scratch_matches_workspace_entry_point(gpu):
    L = lib()
    assert L.eet_mmha_decode_static_capacity() >= 512 * 130 * 4
    # first call: B*H = 32 < 256 at step 1024 -> the time axis is split (workspace needed by the
    # existing entry point); second call, smaller: B*H = 8 at step 600, with ALiBi and padding;
    # third: no split at all (B*H = 256), the array is not touched
    for seed, (B, H, dh, step, alibi, pad) in enumerate([(1, 32, 128, 1024, False, None),
                                                         (2, 4, 64, 600, True, [0, 17]),
                                                         (8, 32, 128, 300, False, None)]):
        assert (L.eet_mmha_decode_workspace(B, H, dh, step) > 0) == (seed < 2)
        q, k, v, kc, vc, bias, padt = case(gpu, seed, B, H, dh, step, alibi, pad)
        kc2, vc2 = kc.clone(), vc.clone()
        print(f"static decode attention: B={B} H={H} dh={dh} step={step}", flush=True)
        want = mmha(q, k, v, kc, vc, step, pad=padt, alibi=bias)
        got = static_call(q, k, v, kc2, vc2, step, pad=padt, alibi=bias)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(kc2, kc) and torch.equal(vc2, vc)          # the appended row too


def test_static_scratch_rejects_oversized_split(gpu, tuning):
    B, H, dh, step = 8, 32, 128, 4096
    q, k, v, kc, vc, _, _ = case(gpu, 5, B, H, dh, step)
    tuning("EET_MMHA_NSPLIT", 4)                  # 256 * 4 records > 512
    with pytest.raises(RuntimeError, match="exceed the static scratch"):
        static_call(q, k, v, kc, vc, step)
    tuning("EET_MMHA_NSPLIT", 2)                  # 512 records: exactly the capacity
    got = static_call(q, k, v, kc.clone(), vc.clone(), step)
    want = mmha(q, k, v, kc, vc, step)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
