"""The adaptive speculation policy (host logic of the generation loop) against the value cases the reference's
own tests hold (crates/qwen-cli/src/qwen/tests.rs:300-530): gate functions, prefix replay, the long-context
acceptance / fallback bands, probe pricing and sustained re-entry, and the short-context window.  Runs without a
GPU: the functions are plain host code of the library."""
import ctypes as C

import pytest

import qwen_llm_amd as dfl

OFF_CTX = 16384
NONE, ACCEPTANCE, FALLBACK = 0, 1, 2


@pytest.fixture(scope="module")
def L():
    return dfl.adaptive_lib()


def new_state(L, reason=NONE, long_mode=False):
    s = dfl.AdaptiveStateC()
    L.dflash_adaptive_init(C.byref(s))
    s.reason, s.long_mode = reason, int(long_mode)
    return s


def record_long(L, s, n_accepted, fallback_ran, was_probe):
    L.dflash_adaptive_prepare_mode(C.byref(s), 1)
    L.dflash_adaptive_record_spec_step(C.byref(s), n_accepted, int(fallback_ran), int(was_probe), 1, 0, 1, 64000)


def test_serial_tail_when_a_full_block_will_not_fit(L):
    """tests.rs:301-327"""
    for remaining in range(8):
        assert not L.dflash_speculation_enabled(0, 100, OFF_CTX, remaining, 8, 0, 0)
    assert L.dflash_speculation_enabled(0, 100, OFF_CTX, 8, 8, 0, 0)
    assert not L.dflash_speculation_enabled(0, 100, OFF_CTX, 8, 8, 1, 0)
    assert L.dflash_speculation_enabled(0, 100, OFF_CTX, 8, 8, 1, 1)
    assert not L.dflash_speculation_enabled(0, OFF_CTX, OFF_CTX, 8, 8, 0, 0)
    assert not L.dflash_speculation_enabled(1, 100, OFF_CTX, 8, 8, 0, 0)


def test_prefix_replay_requires_an_exact_emitted_prefix(L):
    """tests.rs:331-398"""
    history = (C.c_int32 * 12)(*range(10, 22))

    def drafts(emitted, k):
        e = (C.c_int32 * max(len(emitted), 1))(*emitted)
        out = C.POINTER(C.c_int32)()
        ok = L.dflash_prefix_replay_drafts(history, 12, e, len(emitted), k, C.byref(out))
        return [out[i] for i in range(k)] if ok else None

    assert drafts([10, 11], 7) == [12, 13, 14, 15, 16, 17, 18]
    assert drafts([10, 99], 7) is None
    assert drafts(list(range(10, 17)), 7) is None  # only five tokens left behind the prefix
    assert drafts([10, 11, 12], 7) == list(range(13, 20))
    D = OFF_CTX
    assert L.dflash_prefix_replay_allowed(0, 100, D, 8, 8, 0, 0, 0)
    assert not L.dflash_prefix_replay_allowed(1, 100, D, 8, 8, 0, 0, 0)
    assert not L.dflash_prefix_replay_allowed(0, D, D, 8, 8, 0, 0, 0)
    assert not L.dflash_prefix_replay_allowed(0, 100, D, 7, 8, 0, 0, 0)
    assert L.dflash_prefix_replay_allowed(0, 100, D, 8, 8, 0, 1, 0)
    assert L.dflash_prefix_replay_allowed(0, 20000, 65536, 8, 8, 1, 1, 1)
    assert not L.dflash_prefix_replay_allowed(0, 20000, 65536, 8, 8, 1, 1, 0)


def test_long_policy_separates_measured_acceptance_bands(L):
    """tests.rs:418-436"""
    losing = new_state(L)
    for a in [2] * 9 + [1] * 7:
        record_long(L, losing, a, False, False)
    assert losing.reason == ACCEPTANCE
    winning = new_state(L)
    for a in [3] * 7 + [2] * 9:
        record_long(L, winning, a, False, False)
    assert winning.reason == NONE
    strong = new_state(L)
    for a in [5] * 15 + [4]:
        record_long(L, strong, a, False, False)
    assert strong.reason == NONE


def test_long_policy_backs_off_on_dense_exact_fallback(L):
    """tests.rs:439-463"""
    cases = [(1, [True, False, True, False], FALLBACK), (4, [True, False, True, False], NONE),
             (4, [True, False] * 4, FALLBACK), (4, [True, False, True, False, True, False, False, False], NONE)]
    for accepted, pattern, want in cases:
        s = new_state(L)
        for f in pattern:
            record_long(L, s, accepted, f, False)
        assert s.reason == want, (accepted, pattern)


def test_long_policy_prices_probes_and_requires_sustained_reentry(L):
    """tests.rs:466-517"""
    acc = new_state(L, ACCEPTANCE, True)
    for _ in range(63):
        L.dflash_adaptive_record_off_step(C.byref(acc))
    assert not L.dflash_adaptive_probe_due(C.byref(acc), 0, 1)
    L.dflash_adaptive_record_off_step(C.byref(acc))
    assert L.dflash_adaptive_probe_due(C.byref(acc), 0, 1)

    fb = new_state(L, FALLBACK, True)
    for _ in range(256):
        L.dflash_adaptive_record_off_step(C.byref(fb))
    assert L.dflash_adaptive_probe_due(C.byref(fb), 0, 1)
    record_long(L, fb, 2, False, True)
    assert fb.reason == FALLBACK
    record_long(L, fb, 3, False, True)
    assert fb.reason == NONE

    interrupted = new_state(L, ACCEPTANCE, True)
    record_long(L, interrupted, 4, False, True)
    record_long(L, interrupted, 4, True, True)
    record_long(L, interrupted, 4, False, True)
    assert interrupted.reason == FALLBACK

    replay_only = new_state(L, ACCEPTANCE, True)
    for _ in range(2):
        L.dflash_adaptive_record_spec_step(C.byref(replay_only), 7, 0, 1, 0, 0, 1, 64000)
    assert replay_only.reason == ACCEPTANCE and replay_only.n_reentry == 0


def test_fallback_density_does_not_change_short_context_policy(L):
    """tests.rs:520-526"""
    s = new_state(L)
    for _ in range(8):
        L.dflash_adaptive_record_spec_step(C.byref(s), 4, 1, 0, 1, 0, 0, 8000)
    assert s.reason == NONE


def test_short_context_window_break_even_and_probe_intervals(L):
    """qwen/dflash.rs:341-352, 206-219: the window must be full; mean emitted below 3.1 - 0.6 turns speculation off,
    a later full window at or above it turns it back on; probes every 8 off steps (32 when sampling)."""
    s = new_state(L)
    for _ in range(15):
        L.dflash_adaptive_record_spec_step(C.byref(s), 1, 0, 0, 1, 0, 0, 500)
    assert s.reason == NONE  # 15 of 16
    L.dflash_adaptive_record_spec_step(C.byref(s), 1, 0, 0, 1, 0, 0, 500)
    assert s.reason == ACCEPTANCE and L.dflash_adaptive_backoff_active(C.byref(s))  # mean emitted 2.0 < 2.5
    assert not L.dflash_adaptive_probe_due(C.byref(s), 0, 0)  # no off step yet
    for i in range(1, 9):
        L.dflash_adaptive_record_off_step(C.byref(s))
        assert bool(L.dflash_adaptive_probe_due(C.byref(s), 0, 0)) == (i == 8)
        assert not L.dflash_adaptive_probe_due(C.byref(s), 1, 0)  # sampled: every 32
    L.dflash_adaptive_begin_spec_step(C.byref(s))
    assert s.off_steps_since_probe == 0
    for _ in range(12):  # the window slides: 4 x 1 and 12 x 2 -> mean emitted 2.75 >= 2.5
        L.dflash_adaptive_record_spec_step(C.byref(s), 2, 0, 1, 1, 0, 0, 500)
    assert s.reason == NONE
    t = new_state(L)
    for _ in range(8):  # sampled: window of 8; mean emitted exactly 2.5 is not below the threshold
        L.dflash_adaptive_record_spec_step(C.byref(t), 1, 0, 0, 1, 1, 0, 500)
    assert t.reason == ACCEPTANCE
    u = new_state(L)
    for a in [1, 2] * 4:
        L.dflash_adaptive_record_spec_step(C.byref(u), a, 0, 0, 1, 1, 0, 500)
    assert u.reason == NONE  # mean emitted 2.5
    assert abs(L.dflash_verify_fallback_margin(100) - 0.1) < 1e-7 and abs(L.dflash_verify_fallback_margin(OFF_CTX) - 0.75) < 1e-7
