"""The C-ABI library loads, exports every symbol include/ucm_hip.h declares,
and rejects bad arguments on the host before anything reaches a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ucm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ucm_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_path():
    syms = declared_symbols()
    for must in ["ucm_block_mean", "ucm_score_blocks", "ucm_topk_windows", "ucm_copy_batch",
                 "ucm_kv_gather_blocks", "ucm_kv_scatter_blocks", "ucm_kv_gather_selected"]:
        assert must in syms


def test_library_exports_every_declared_symbol(ucm):
    from ucm_amd import _lib

    lib = C.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in include/ucm_hip.h but not exported"
    # and the python binding knows each of them
    assert set(declared_symbols()) == set(_lib.SIGNATURES)
    assert _lib.lib().ucm_version() >= 100


def test_bad_arguments_fail_on_the_host(ucm):
    from ucm_amd import _lib

    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_copy_batch", None, None, 4, 64, None)
    assert e.value.code == _lib.EINVAL and "null" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_copy_batch", 16, 16, 4, 24, None)  # size not a multiple of 16
    assert e.value.code == _lib.EINVAL
    _lib.call("ucm_copy_batch", None, None, 0, 64, None)  # an empty batch is a no-op, pointers unchecked
    # head_dim the scoring kernel was not built for
    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_score_blocks", 16, 0, 0, None, 32, 16, 0, 0, 8, 1, 16, 16, 1, 8, 0, 1, 8, 80, 16, 0, 1.0, 0, None)
    assert e.value.code == _lib.ENOTSUP and "head_dim" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_score_blocks", 16, 0, 0, None, 30, 16, 0, 0, 8, 1, 16, 16, 1, 8, 0, 1, 6, 128, 16, 0, 1.0, 0, None)
    assert e.value.code == _lib.ENOTSUP and "kv_heads" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:  # two representatives for each of 16 heads: more vectors per block than a pass holds
        _lib.call("ucm_score_blocks", 16, 0, 0, None, 32, 16, 0, 0, 8, 2, 16, 16, 1, 8, 0, 1, 16, 64, 16, 0, 1.0, 0, None)
    assert e.value.code == _lib.ENOTSUP and "num_repre" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:  # layers closer together than the rows the call names
        _lib.call("ucm_score_blocks", 16, 0, 0, None, 32, 16, 0, 1024, 8, 1, 16, 16, 1, 8, 0, 2, 8, 128, 16, 8, 1.0, 0, None)
    assert e.value.code == _lib.EINVAL and "repre_rows" in str(e.value)
    # the one-launch entry point: an argument block of another size, requests longer than its selection holds
    args = _lib.ScoreSelectArgs()
    args.struct_size = 8
    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_score_select", C.addressof(args), None)
    assert e.value.code == _lib.EINVAL and "struct_size" in str(e.value)
    args = _lib.ScoreSelectArgs(q=16, q_heads=32, repre=16, repre_rows=8, seg_off=16, seg_len=16, topk_len=16, n_req=1,
                                max_seg_len=2000, kv_heads=8, head_dim=128, scores=16, idx_out=16, count_out=16,
                                out_stride=2000, tickets=16)
    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_score_select", C.addressof(args), None)
    assert e.value.code == _lib.ENOTSUP and "1024" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:  # a workspace smaller than the call's path stores through
        _lib.call("ucm_kvstar_votes", 16, 1 << 20, 16, 8, 32, 128, None, 0, None, 16, 400, 1024 * 100, 1024, 16, 16, 4, 100, 8, 8,
                  128, 128, 16, 1, 16, 1, 16, 0, None)
    assert e.value.code == _lib.EINVAL and "workspace" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:  # more blocks per request than the selection kernel holds
        _lib.call("ucm_topk_windows", 16, 0, 5000, 16, 16, 16, 1, 5000, 1, 1, 2, 16, 5000, 16, None, 0, None, None, 0, None, None)
    assert e.value.code == _lib.ENOTSUP
    with pytest.raises(_lib.UcmHipError) as e:  # output row too short for the identity path
        _lib.call("ucm_topk_windows", 16, 0, 100, 16, 16, 16, 1, 100, 1, 1, 2, 16, 50, 16, None, 0, None, None, 0, None, None)
    assert e.value.code == _lib.EINVAL and "out_stride" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:  # block does not fit the plane stride
        _lib.call("ucm_kv_gather_blocks", 16, 2, 1024, 512, 4, 16, 1, 16, None)
    assert e.value.code == _lib.EINVAL and "num_blocks" in str(e.value)
    with pytest.raises(_lib.UcmHipError) as e:
        _lib.call("ucm_block_mean", 16, 1, 8, 16, 16, 1, 128, 3, 3, 16, 8, 0, 0, None)  # row of 9 columns
    assert e.value.code == _lib.ENOTSUP
    with pytest.raises(_lib.UcmHipError) as e:  # more candidate scores than the built-in scratch holds
        _lib.call("ucm_esa_retrieve_static", 16, 100, 1024, 16, 16, 65, 8192, 4, 16, 16, 16, 4, None)
    assert e.value.code == _lib.ENOTSUP and "scratch" in str(e.value)


def test_ops_need_device_tensors(ucm):
    import torch

    from ucm_amd import ops

    with pytest.raises(ValueError):
        ops.copy_batch(torch.zeros(2, dtype=torch.int64), torch.zeros(2, dtype=torch.int64), 16)


def test_missing_library_is_loud(ucm, monkeypatch):
    from ucm_amd import _lib

    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libucm_hip.so")
    with pytest.raises(ImportError, match="no CPU fallback"):
        _lib.load()
