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


def test_native_module_binds_the_reference_names():
    """`infllm_v2.C` is the compiled extension and exports what csrc/entry.cu:197-215 binds; argument errors that need
    no GPU are reported on the host."""
    import pytest
    import torch
    from infllm_v2 import C
    import infllmv2_cuda_impl_amd._C as ext
    names = ["topk", "get_probs", "blockmask_to_uint64", "topk_to_uint64", "uint64_to_bool", "max_pooling_1d",
             "max_pooling_1d_varlen", "fwd", "varlen_fwd", "varlen_fwd_stage1", "bwd", "varlen_bwd", "fwd_kvcache"]
    for n in names:
        assert getattr(C, n) is getattr(ext, n), n
    with pytest.raises(NotImplementedError):
        C.get_probs()
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16)
    cu = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        C.varlen_fwd(z(4, 32, 128), z(4, 2, 128), z(4, 2, 128), None, cu, cu, None, None, None, None, 4, 4, 0.0, 0.088,
                     False, True, -1, -1, 0.0, False, None, None)
    with pytest.raises(RuntimeError, match="same dtype"):
        C.varlen_fwd(z(4, 32, 128), z(4, 2, 128).float(), z(4, 2, 128), None, cu, cu, None, None, None, None, 4, 4, 0.0,
                     0.088, False, True, -1, -1, 0.0, False, None, None)
    with pytest.raises(RuntimeError, match="does not support softcap"):
        C.fwd_kvcache(z(1, 1, 32, 128), z(1, 64, 2, 128), z(1, 64, 2, 128), None, None, None, None, None, None, None, None,
                      None, None, 0.088, False, -1, -1, 1.0, True, 0, None)
