"""Learning-rate schedulers (host arithmetic of libboat_amd.so; no GPU work): bit-exact against the compiled reference
where it was built, against the closed forms of src/schedulers/*.c always, and the reference's own checks
(tests/unit/test_schedulers.c) on both."""
import ctypes as C
import math

import numpy as np
import pytest

import boat_cases as bc


@pytest.fixture(scope="module")
def amd():
    from boat_amd.capi import BoatAPI
    return BoatAPI()          # loading needs no GPU; the scheduler entry points never touch the device


def lam(step, base):
    return base / (1.0 + 0.1 * step) if step < 12 else -1.0        # negative values are clamped to 0 (lambda_lr.c:52-54)


CASES = [("step", 0.1, 25, dict(step_size=10, gamma=0.5)), ("step", 1e-3, 7, dict(step_size=1, gamma=0.9)),
         ("cosine", 0.1, 130, dict(T_max=100, eta_min=0.001)), ("cosine", 3e-4, 9, dict(T_max=4, eta_min=0.0)),
         ("lambda", 0.05, 15, dict(fn=lam))]


@pytest.mark.parametrize("kind,base,steps,kw", CASES, ids=lambda v: v if isinstance(v, str) else None)
def test_scheduler_matches_compiled_reference_bit_for_bit(ref, amd, kind, base, steps, kw):
    got = bc.scheduler_trajectory(amd, kind, base, steps, **kw)
    want = bc.scheduler_trajectory(ref, kind, base, steps, **kw)
    assert got.shape == want.shape and np.array_equal(got, want)


def test_scheduler_closed_forms_and_reference_unit_checks(amd):
    # tests/unit/test_schedulers.c: StepLR(0.1, 10, 0.5): 0.1 for steps 1..10, 0.05 for 11..20, 0.025 after
    t = bc.scheduler_trajectory(amd, "step", 0.1, 25, step_size=10, gamma=0.5)
    assert t[0].tolist() == [np.float32(0.1)] * 2                              # before the first step: base rate
    for step in range(1, 26):
        want = np.float32(0.1) * np.float32(0.5) ** ((step - 1) // 10)
        assert abs(t[step][1] - want) <= 1e-7 and t[step][0] == t[step][1]     # next_lr previews what step() sets
    assert t[-1].tolist() == [np.float32(0.1)] * 2                             # reset
    # cosine: eta_min + (base-eta_min)/2 * (1 + cos(pi*min(t,T)/T)); stays at eta_min after T_max
    t = bc.scheduler_trajectory(amd, "cosine", 0.1, 130, T_max=100, eta_min=0.001)
    for step in (1, 50, 100, 130):
        want = 0.001 + 0.5 * (0.1 - 0.001) * (1 + math.cos(math.pi * min(step, 100) / 100))
        assert abs(t[step][1] - want) <= 2e-7
    assert abs(t[50][1] - (0.1 + 0.001) / 2) <= 1e-6 and abs(t[130][1] - 0.001) <= 1e-7
    assert np.all(np.diff(t[1:101, 1]) <= 0)                                   # monotone decay up to T_max
    t = bc.scheduler_trajectory(amd, "lambda", 0.05, 15, fn=lam)
    assert abs(t[3][1] - 0.05 / 1.3) <= 1e-8 and t[12][1] == 0 and t[15][1] == 0
    # argument validation (step_lr.c:20-30, cosine_annealing.c:20-33, lambda_lr.c:19-25)
    assert bc.scheduler_trajectory(amd, "step", 0.0, 1, step_size=1, gamma=0.5) is None
    assert bc.scheduler_trajectory(amd, "step", 0.1, 1, step_size=0, gamma=0.5) is None
    assert bc.scheduler_trajectory(amd, "step", 0.1, 1, step_size=1, gamma=0.0) is None
    assert bc.scheduler_trajectory(amd, "cosine", 0.1, 1, T_max=0, eta_min=0.0) is None
    assert bc.scheduler_trajectory(amd, "cosine", 0.1, 1, T_max=5, eta_min=0.1) is None
    assert bc.scheduler_trajectory(amd, "cosine", 0.1, 1, T_max=5, eta_min=-0.1) is None
    from boat_amd.capi import LAMBDA_LR_FN
    assert not amd.boat_lambda_lr_scheduler_create(0.1, C.cast(None, LAMBDA_LR_FN))
    assert amd.boat_scheduler_get_last_lr(None) == 0 and amd.boat_scheduler_get_next_lr(None) == 0
    amd.boat_scheduler_step(None)
    amd.boat_scheduler_free(None)


@pytest.mark.gpu
def test_scheduler_drives_the_optimizer(boat):
    """boat_scheduler_update_optimizer hands the rate to Adam; the next step moves the parameter by that rate
    (first Adam step from zero moments: |dp| = lr * |g| / (|g| + eps))."""
    p = boat.tensor(np.array([5.0, -3.0], np.float32))
    g = boat.tensor(np.array([2.0, 0.5], np.float32))
    opt = boat.boat_adam_optimizer_create(0.5, 0.9, 0.999, 1e-8)
    boat.boat_optimizer_add_parameter(opt, p, g)
    s = boat.boat_step_lr_scheduler_create(0.01, 1, 0.1)
    boat.boat_scheduler_step(s)
    boat.boat_scheduler_step(s)                      # rate 0.001
    boat.boat_scheduler_update_optimizer(s, opt)
    assert abs(boat.boat_optimizer_get_learning_rate(opt) - 0.001) <= 1e-9
    boat.boat_optimizer_step(opt)
    assert np.allclose(boat.numpy(p), [5.0 - 0.001, -3.0 - 0.001], rtol=0, atol=1e-6)
    boat.boat_scheduler_update_optimizer(None, opt)  # no-ops
    boat.boat_scheduler_update_optimizer(s, None)
    boat.boat_scheduler_free(s)
    boat.boat_optimizer_free(opt)
    boat.boat_tensor_unref(p)
    boat.boat_tensor_unref(g)
