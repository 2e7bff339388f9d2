"""CPU-side checks: the built library exports every symbol the C header declares (no compute calls), the host
metadata logic, and the config validation."""
import ctypes
import os

import pytest
import torch


def test_library_exports_every_declared_symbol():
    from flash_nsa import _lib
    protos = _lib.parse_header()
    assert len(protos) >= 25
    assert os.path.exists(_lib.LIB_PATH), "libnsa_hip.so is not built (run __graft_entry__.build())"
    dll = ctypes.CDLL(_lib.LIB_PATH)
    for name in protos:
        assert hasattr(dll, name), f"{name} is declared in include/nsa_hip.h but not exported"
    dll.nsa_abi_version.restype = ctypes.c_int
    assert dll.nsa_abi_version() >= 1


def test_entry_points_reject_bad_arguments_without_a_gpu():
    from flash_nsa import _lib
    with pytest.raises(RuntimeError, match="multiple of 8"):
        _lib.call("nsa_mean_pool_fwd", None, 0, 0, None, 0, 0, None, None, 1, 1, 1, 12, 32, 16, None)
    with pytest.raises(RuntimeError, match="power of 2"):
        _lib.call("nsa_cmp_attn_fwd", None, 0, 0, None, 0, 0, None, 0, 0, None, 0, 0, None, 0, 0, None, None, 1, 8, 16,
                  1, 128, 128, 32, 12, 1.0, None)
    with pytest.raises(RuntimeError, match="kv heads"):
        _lib.call("nsa_swa_fwd", None, 0, 0, None, 0, 0, None, 0, 0, None, 0, 0, None, 0, 0, None, 1, 8, 16, 3, 128,
                  128, 512, 1.0, None)
    with pytest.raises(RuntimeError, match="unsupported head dims"):
        _lib.call("nsa_swa_fwd", None, 0, 0, None, 0, 0, None, 0, 0, None, 0, 0, None, 0, 0, None, 1, 8, 16, 1, 96,
                  96, 512, 1.0, None)


def test_nsa_helper_metadata():
    from flash_nsa import NSAHelper
    NSAHelper.set_hyperparameters()
    cu = torch.tensor([0, 31, 63, 163, 163, 4259], dtype=torch.int32)
    NSAHelper.init_cu_seqlens(cu)
    assert NSAHelper.batch == 5
    assert NSAHelper.x_maxlen == 4096
    assert NSAHelper.y_seqlens.tolist() == [0, 1, 5, 0, 255]
    assert NSAHelper.y_cu_seqlens.tolist() == [0, 0, 1, 6, 6, 261]
    assert NSAHelper.k_seqlens.tolist() == [1, 1, 2, 0, 64]
    assert NSAHelper.k_len == 68 and NSAHelper.y_len == 261 and NSAHelper.y_maxlen == 255
    assert NSAHelper.blk_seq.tolist() == [0, 1, 2, 2] + [4] * 64
    # changing the hyper-parameters invalidates the cached batch
    NSAHelper.set_hyperparameters(kernel_size=64, stride=32, block_size=128)
    NSAHelper.init_cu_seqlens(cu)
    assert NSAHelper.y_seqlens.tolist() == [0, 0, 2, 0, 127]
    NSAHelper.set_hyperparameters()


def test_config_validation(tmp_path):
    from flash_nsa import NSAConfig
    c = NSAConfig(head_dim=64)
    assert c.qk_head_dim == 64 and c.v_head_dim == 64
    with pytest.raises(AssertionError):
        NSAConfig(stride=12)
    with pytest.raises(AssertionError):
        NSAConfig(kernel_size=40)
    with pytest.raises(AssertionError):
        NSAConfig(block_size=16)
    p = tmp_path / "c.json"
    p.write_text('{"num_heads": 32, "top_n": 8, "slc_block_size": 64}')
    c = NSAConfig.from_json(str(p))
    assert c.num_heads == 32 and c.top_n == 8 and c.slc_block_size == 64


def test_bench_flop_model_matches_closed_form():
    import bench
    nc, ns, nw = bench.branch_counts([65536])
    assert (nc, ns, nw) == (134123535, 66617344, 33488640)
    f = bench.stage_flops([65536], 64, 128, 128)
    assert abs(f["fwd_total"] / 1e12 - 9.87) < 0.01
    assert abs(f["bwd_total"] / 1e12 - 19.19) < 0.01


def test_helper_does_not_confuse_a_new_tensor_with_the_registered_one():
    """A second cu_seqlens tensor with other lengths must be re-registered even when it is as long as the first one
    (an allocator may even hand it the same address); the same unmodified object is recognised without a read."""
    import torch
    from flash_nsa import NSAHelper
    NSAHelper.set_hyperparameters()
    a = torch.tensor([0, 700, 960], dtype=torch.int32)
    NSAHelper.init_cu_seqlens(a)
    assert (NSAHelper.x_maxlen, NSAHelper.y_len) == (700, 42 + 15)
    del a
    b = torch.tensor([0, 400, 730], dtype=torch.int32)
    NSAHelper.init_cu_seqlens(b)
    assert (NSAHelper.x_maxlen, NSAHelper.y_len) == (400, 24 + 19)
    NSAHelper.init_cu_seqlens(b)
    assert NSAHelper.x_maxlen == 400
    b[1] = 330                      # in-place edit of the registered tensor bumps its version
    NSAHelper.init_cu_seqlens(b)
    assert (NSAHelper.x_maxlen, NSAHelper.y_len) == (400, 19 + 24)
    assert NSAHelper._host_cu == [0, 330, 730]


def test_split_decode_lds_budget_counts_static_arrays():
    """nsa_decode_split_fits must imply dynamic + statically declared LDS <= 160 KB for the second launch: a
    capacity whose dynamic part alone fits but whose total does not has to be reported as not fitting, so that
    nsa_decode falls back instead of failing at launch.  Host arithmetic only."""
    from flash_nsa import _lib
    limit = 160 * 1024
    seen_near_limit = 0
    for D in (128, 64):
        for y in (512, 2048, 8192, 16384, 20000, 20480, 24576, 32768):
            for nb in (64, 512, 2048, 4096, 8192):
                prev_fit = True
                for tw in list(range(8, 6000, 97)):
                    fits = _lib.value("nsa_decode_split_fits", D, D, y, nb, tw)
                    total = _lib.value("nsa_decode_split_lds_total", D, D, y, nb, tw)
                    assert (total > 0) == bool(fits)
                    if fits:
                        assert 4288 < total <= limit, (D, y, nb, tw, total)
                        assert prev_fit, "a wider table cannot fit where a narrower one did not"
                        seen_near_limit += total > limit - 4288
                    prev_fit = bool(fits)
    assert seen_near_limit > 0, "the sweep must reach totals within the static part of the limit"


def test_inverse_index_refuses_more_blocks_than_its_histogram_holds():
    """The inverse index counts per selection block in an LDS histogram of 16384 entries: a batch with more blocks
    (more than 1048576 tokens at 64 per block) is refused with a message instead of launched."""
    from flash_nsa import _lib
    with pytest.raises(RuntimeError, match="exceed the LDS histogram"):
        _lib.call("nsa_build_inverse_index", None, 0, 0, 16, None, None, 1, 1 << 21, 4, 16385, 64, 1024, None, None,
                  None, None, 0, None)


def test_tuning_values_are_set_by_name_not_by_environment():
    from flash_nsa import _lib
    _lib.call("nsa_set_tuning", b"topk_seg_blocks", 64)
    _lib.call("nsa_reset_tuning")
    with pytest.raises(RuntimeError, match="unknown name"):
        _lib.call("nsa_set_tuning", b"no_such_value", 1)


def test_unsupported_shapes_are_rejected_where_the_model_is_configured():
    """Block sizes that are not multiples of 32 and head dims that are not built fail in NSAConfig and in both
    cores' constructors (also for a plain attribute object), not at the first launch in the middle of a forward."""
    from types import SimpleNamespace
    from flash_nsa import NSAConfig, NSACore, HFNSACore
    NSAConfig(block_size=32)
    NSAConfig(block_size=256, kernel_size=64)
    NSAConfig(qk_head_dim=192, v_head_dim=128)
    with pytest.raises(AssertionError, match="multiples of 32"):
        NSAConfig(block_size=48)
    NSAConfig(head_dim=256)
    NSAConfig(head_dim=32)
    with pytest.raises(AssertionError, match="not built"):
        NSAConfig(head_dim=512)
    with pytest.raises(AssertionError, match="not built"):
        NSAConfig(qk_head_dim=256, v_head_dim=128)
    loose = SimpleNamespace(head_dim=128, qk_head_dim=None, v_head_dim=None, num_heads=16, num_kv_heads=1,
                            kernel_size=32, stride=16, block_size=80, cmp_k_method="mean", cmp_v_method="mean")
    for core in (NSACore, HFNSACore):
        with pytest.raises(AssertionError, match="multiples of 32"):
            core(loose)
    loose.block_size, loose.head_dim = 64, 96
    for core in (NSACore, HFNSACore):
        with pytest.raises(AssertionError, match="not built"):
            core(loose)
