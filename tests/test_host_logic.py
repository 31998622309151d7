"""Host-side argument logic that needs no GPU."""
import pytest


def test_causal_flag_is_derived_from_the_window_as_in_the_reference():
    """flash_api.cpp:621-622 (a window side >= max_seqlen_k is unbounded), :600 (causal closes the right side),
    :137 (causal launch iff left unbounded and right == 0), :144-147 (anything else is local attention: rejected)."""
    from infllmv2_cuda_impl_amd.attention import normalise_causal as f
    assert f(True, (-1, -1)) is True
    assert f(False, (-1, -1)) is False
    assert f(False, (-1, 0)) is True                       # the case an int(bool(causal)) launch gets wrong
    assert f(True, (-1, 5)) is True                        # causal overrides the right side
    assert f(False, (-1, 5)) is None
    assert f(False, (7, 0)) is None and f(True, (7, -1)) is None
    assert f(False, (128, 0), max_seqlen_k=128) is True    # left side reaches the keys: unbounded
    assert f(False, (127, 0), max_seqlen_k=128) is None
    assert f(False, (500, 500), max_seqlen_k=128) is False
    assert f(False, (-1, 128), max_seqlen_k=128) is False
    assert f(False, (128, 0)) is None                      # without max_seqlen_k nothing is widened


def test_reject_unsupported_returns_the_launch_flag_and_keeps_the_reference_messages():
    from infllmv2_cuda_impl_amd.attention import _reject_unsupported as r
    assert r(0.0, (-1, 0), 0.0, None, False, 64) is True
    assert r(0.0, (-1, -1), 0.0, None, False, 64) is False
    with pytest.raises(RuntimeError, match="does not support local attention"):
        r(0.0, (3, 0), 0.0, None, False, 64)
    with pytest.raises(RuntimeError, match="does not support softcap"):
        r(0.0, (-1, -1), 1.0, None, True, 64)
    with pytest.raises(RuntimeError, match="does not support dropout"):
        r(0.5, (-1, -1), 0.0, None, True, 64)
    with pytest.raises(RuntimeError, match="does not support alibi"):
        r(0.0, (-1, -1), 0.0, object(), True, 64)
