"""The loss-scale schedule on the device (``rg_scaler_init`` / ``rg_scaler_update``) against the
oracle's restatement of Apex's ``LossScaler.update_scale`` and of the reference's wrapper around it
(``pyrannc/amp/__init__.py:44-65``), step by step over seeded overflow sequences.  The result
block the schedule reads is written by the test itself, so every branch is reached: floor, cap,
integer truncation, window doubling right after an overflow, a static scale."""
import ctypes as C
import random
import zlib

import pytest
import torch

import oracle.gradpath as oracle
from rannc_amd import _lib
from rannc_amd.multi_tensor import stream_handle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

# rg_step_result: double norm; float coef; int overflow, clipped, skipped
RESULT_OVERFLOW_WORD = 3


def _read_state(state: torch.Tensor) -> _lib.ScalerState:
    torch.cuda.synchronize()
    raw = bytes(state.cpu().numpy().tobytes())
    return _lib.ScalerState.from_buffer_copy(raw[:C.sizeof(_lib.ScalerState)])


CASES = [
    # name, init scale, min, max, window, dynamic, truncate, P(overflow)
    ("apex_default_window_3", 2.0 ** 16, None, 2.0 ** 24, 3, True, False, 0.3),
    ("reference_wrapper_truncates", 50000.0, None, 2.0 ** 24, 2, True, True, 0.3),
    ("floor_reached", 8.0, 2.0, 2.0 ** 24, 4, True, False, 0.7),
    ("floor_not_an_integer_then_truncated", 9.0, 2.5, 2.0 ** 24, 5, True, True, 0.7),
    ("cap_reached", 2.0 ** 22, None, 2.0 ** 24, 1, True, False, 0.1),
    ("window_one_doubles_every_clean_step", 3.0, 1.0, 48.0, 1, True, True, 0.25),
    ("static_never_moves", 128.0, None, 2.0 ** 24, 2, False, False, 0.5),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_device_schedule_follows_the_oracle(case):
    name, scale, floor, cap, window, dynamic, truncate, p_overflow = case
    rng = random.Random(zlib.crc32(name.encode()))
    want = oracle.LossScalerState(loss_scale=scale, unskipped=0, scale_window=window, min_loss_scale=floor,
                                  max_loss_scale=cap, dynamic=dynamic)
    state = torch.zeros(_lib.SCALER_STATE_BYTES, dtype=torch.uint8, device=DEV)
    result = torch.zeros(8, dtype=torch.int32, device=DEV)
    s = stream_handle(DEV)
    _lib.scaler_init(state.data_ptr(), scale, floor or 0.0, cap, window, 2.0, 0, s)
    got = _read_state(state)
    assert (got.loss_scale, got.unskipped, got.skipped_steps) == (scale, 0, 0)
    assert got.inv_scale == torch.tensor(1.0 / scale, dtype=torch.float32).item()

    flags = (_lib.RG_SCALER_DYNAMIC if dynamic else 0) | (_lib.RG_SCALER_TRUNCATE if truncate else 0)
    skipped_steps = 0
    for step in range(40):
        overflow = rng.random() < p_overflow
        result[RESULT_OVERFLOW_WORD] = 1 if overflow else 0
        if truncate:
            skipped = oracle.patched_update_scale(want, overflow)
        else:
            skipped = want.update_scale(overflow)
        skipped_steps += 1 if skipped else 0
        _lib.scaler_update(state.data_ptr(), result.data_ptr(), flags, 0, s)
        got = _read_state(state)
        assert (got.loss_scale, got.unskipped) == (float(want.loss_scale), want.unskipped), f"{name}: step {step}"
        assert got.skipped_steps == skipped_steps, f"{name}: step {step}"
        # 1/scale is the fp32 rounding of the double quotient: what the host path passes by value
        assert got.inv_scale == torch.tensor(1.0 / float(want.loss_scale), dtype=torch.float32).item()
        if want.loss_scale < 2:     # the reference's truncation would reach zero next: nothing left to compare
            break
    if not dynamic:
        assert skipped_steps == 0 and got.loss_scale == scale


def test_update_rejects_null_pointers():
    state = torch.zeros(_lib.SCALER_STATE_BYTES, dtype=torch.uint8, device=DEV)
    with pytest.raises((ValueError, RuntimeError)):
        _lib.scaler_update(state.data_ptr(), 0, _lib.RG_SCALER_DYNAMIC, 0, stream_handle(DEV))
    with pytest.raises((ValueError, RuntimeError)):
        _lib.scaler_update(0, state.data_ptr(), _lib.RG_SCALER_DYNAMIC, 0, stream_handle(DEV))
