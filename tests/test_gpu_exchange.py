"""GPU test of the split-K exchange's give-up path: with the collectors' poll limit forced to zero from the host (every
kernel still runs to its end at once), a launch whose collectors find a partial tile missing writes NaN, raises the flag
that hidet_qmm_exchange_status reports, and may leave stale words in the mailbox; hidet_qmm_exchange_reset puts the
workspace back, and the next launch is bit-exact again."""
import numpy as np
import pytest
import torch

from hidet_amd import ffi
from oracle import clib
from oracle import oracle as O
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu


def _run(a, q, s, ws, parts=0):
    m, k = a.shape
    n = q.shape[1]
    c = torch.zeros((m, n), dtype=torch.float16, device=a.device)
    ffi.call('hidet_symmetric_quant_matmul_f16_i8', a, q, s, c, m, k, n, a.stride(0), parts, ws, ws.numel(),
             ffi.current_stream(a.device))
    return c


def test_lost_partial_is_reported_and_reset_recovers():
    lib = ffi.load_library()
    # 43 column tiles shared by 256 workgroups that all finish their rows at about the same time: a collector's first look
    # at the mailbox comes while some of its five or six senders still store
    m, k, n = 1, 4096, 11008
    a32, w32 = O.make_inputs(7, m, k, n)
    q, s32 = O.symmetric_quantize(w32, 'int8', dims=0)
    a, s = a32.astype(np.float16), s32.astype(np.float16)
    da, dq, ds = dev(a), dev(q), dev(s)
    ws = torch.zeros(int(lib.hidet_qmm_min_workspace_bytes()), dtype=torch.uint8, device='cuda')
    stream = ffi.current_stream(da.device)
    announce('exchange: healthy launch', m, k, n)
    good = host(_run(da, dq, ds, ws))
    assert O.max_rel_err(good, clib.quant_matmul_f32acc(a, q, s)) <= 1e-2
    assert ffi.call('hidet_qmm_exchange_status', ws, ws.numel(), stream) == 0
    assert ffi.call('hidet_qmm_exchange_status', None, 0, stream) == 0  # the static array's

    announce('exchange: poll limit 0')
    lost, bad = 0, None
    lib.hidet_qmm_set_exchange_spin_limit(0)
    try:
        for _ in range(50):  # a collector that happens to find everything there at its first look loses nothing
            bad = host(_run(da, dq, ds, ws))
            lost = ffi.call('hidet_qmm_exchange_status', ws, ws.numel(), stream)
            if lost:
                break
    finally:
        lib.hidet_qmm_set_exchange_spin_limit(-1)
    assert lost == 1, 'no collector gave up in 50 launches with a poll limit of 0'
    # what was not summed is NaN, never a plausible number: every other output is the healthy one
    nan = np.isnan(bad)
    assert nan.any()
    assert np.array_equal(bad[~nan].view(np.uint16), good[~nan].view(np.uint16))
    # the flag is sticky until the reset
    assert ffi.call('hidet_qmm_exchange_status', ws, ws.numel(), stream) == 1

    announce('exchange: reset')
    ffi.call('hidet_qmm_exchange_reset', ws, ws.numel(), stream)
    assert ffi.call('hidet_qmm_exchange_status', ws, ws.numel(), stream) == 0
    mailbox_bytes = min(16 << 20, (ws.numel() - 65536) // 4) // 256 * 256
    assert int(ws[:65536 + mailbox_bytes].max().item()) == 0
    again = host(_run(da, dq, ds, ws))
    assert np.array_equal(again.view(np.uint16), good.view(np.uint16))
    assert ffi.call('hidet_qmm_exchange_status', ws, ws.numel(), stream) == 0
    # the static array takes the same two calls
    ffi.call('hidet_qmm_exchange_reset', None, 0, stream)
    assert ffi.call('hidet_qmm_exchange_status', None, 0, stream) == 0
