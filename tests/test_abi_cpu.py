"""CPU-side checks of the C ABI: the built library loads without a GPU, exports
every symbol ``include/tokenselect.h`` declares, and rejects bad arguments on the
host (before any HIP call) with the documented error codes."""

import ctypes
import os
import re

import pytest
import torch

from tokenselect_amd import _lib, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from tokenselect_amd import build
        build.build(verbose=False)
    return _lib.load()


def cfg(**kw):
    base = dict(num_heads=32, num_kv_heads=8, head_dim=128, page_size=1, n_init=128, n_local=512,
                top_k=2048, pool_kernel=-1, head_map=0, rope_mode=1, rope_theta=5e5, rope_scale=1.0,
                sm_scale=0.088, logit_cap=0.0)
    base.update(kw)
    return _lib.TsConfig(*[base[name] for name, _ in _lib.TsConfig._fields_])


def err(lib):
    return lib.ts_last_error().decode()


def test_header_symbols_are_exported_and_bound(lib):
    header = open(os.path.join(ROOT, "include", "tokenselect.h")).read()
    declared = set(re.findall(r"\b(ts_[a-z_]+)\s*\(", header))
    assert declared, "no declarations found in the header"
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert declared == set(_lib.SIGNATURES), "ctypes signatures and header disagree"
    assert lib.ts_version() == int(re.search(r"#define TS_VERSION (\d+)", header).group(1))


def test_struct_layouts_match_the_header():
    assert ctypes.sizeof(_lib.TsConfig) == 14 * 4
    assert ctypes.sizeof(_lib.TsBatch) == 8 + 8 + 8 + 8 + 8 + 8 + 8 + 8 + 4 * 4 + 8  # 5 ints, padded
    assert _lib.TsBatch.workspace_clean.offset == 80
    assert _lib.TsBatch.threshold_hint.offset == 56
    assert _lib.TsBatch.separate_kernels.offset == 64 and _lib.TsBatch.rerun.offset == 68
    assert _lib.TsBatch.wait_us.offset == 72 and _lib.TsBatch.absent_workgroups.offset == 76
    assert _lib.TsBatch.fault.offset == 40 and _lib.TsBatch.host_seq_lens.offset == 48
    assert _lib.TsBatch.seq_lens.offset == 8 and _lib.TsBatch.table_stride.offset == 24
    assert ctypes.sizeof(_lib.TsSelCache) == 4 * 8 + 8
    assert ctypes.sizeof(_lib.TsNewKv) == 4 * 8 + 8 and _lib.TsNewKv.max_tokens.offset == 32


def test_config_validation(lib):
    assert lib.ts_check_config(ctypes.byref(cfg())) == _lib.TS_OK
    assert lib.ts_check_config(None) == _lib.TS_EINVAL
    assert lib.ts_check_config(ctypes.byref(cfg(head_dim=64))) == _lib.TS_ESHAPE
    assert "head_dim 64" in err(lib)
    assert lib.ts_check_config(ctypes.byref(cfg(num_heads=30))) == _lib.TS_ESHAPE
    assert lib.ts_check_config(ctypes.byref(cfg(num_heads=72, num_kv_heads=8))) == _lib.TS_ESHAPE
    assert lib.ts_check_config(ctypes.byref(cfg(num_heads=24, num_kv_heads=3))) == _lib.TS_ESHAPE
    assert lib.ts_check_config(ctypes.byref(cfg(page_size=12))) == _lib.TS_EINVAL
    assert lib.ts_check_config(ctypes.byref(cfg(top_k=0))) == _lib.TS_EINVAL
    assert lib.ts_check_config(ctypes.byref(cfg(rope_mode=7))) == _lib.TS_EINVAL
    assert lib.ts_check_config(ctypes.byref(cfg(rope_theta=0.0))) == _lib.TS_EINVAL
    for hkv, g in [(1, 8), (2, 2), (4, 7), (8, 4), (8, 8), (4, 1), (8, 3), (2, 6), (4, 5)]:
        assert lib.ts_check_config(ctypes.byref(cfg(num_heads=hkv * g, num_kv_heads=hkv))) == 0


def test_workspace_queries(lib):
    c = cfg()
    assert lib.ts_decode_layer_workspace_bytes(ctypes.byref(c), 1, 131072) > 32 * 131072 * 4
    assert lib.ts_decode_layer_workspace_bytes(ctypes.byref(cfg(head_dim=64)), 1, 1024) == 0
    assert lib.ts_score_partials_bytes(ctypes.byref(c), 1, 131072) % 256 == 0
    assert lib.ts_attn_workspace_bytes(ctypes.byref(c), 4, 2688) > 0


def test_null_and_range_errors_need_no_gpu(lib):
    c = cfg()
    one = ctypes.c_void_p(0x1000)  # never dereferenced: validation fails first
    bt = _lib.TsBatch(1, 4096, one, one, 4096, None)
    assert lib.ts_score(ctypes.byref(c), None, one, one, 10, None, one, 4096, one, 1 << 20,
                        None) == _lib.TS_EINVAL
    assert lib.ts_score(ctypes.byref(c), ctypes.byref(bt), None, one, 10, None, one, 4096, one,
                        1 << 20, None) == _lib.TS_EINVAL
    assert "NULL" in err(lib)
    # score stride smaller than the candidate count
    assert lib.ts_score(ctypes.byref(c), ctypes.byref(bt), one, one, 10, None, one, 100, one,
                        1 << 20, None) == _lib.TS_EWORKSPACE
    # partials buffer too small
    assert lib.ts_score(ctypes.byref(c), ctypes.byref(bt), one, one, 10, None, one, 4096, one, 16,
                        None) == _lib.TS_EWORKSPACE
    bad = _lib.TsBatch(0, 4096, one, one, 4096, None)
    assert lib.ts_vote(ctypes.byref(c), ctypes.byref(bad), one, 4096, one, None, one, one, None,
                       4096, None) == _lib.TS_EINVAL
    # a host-side length beyond max_seq_len
    lens = (ctypes.c_int32 * 1)(5000)
    beyond = _lib.TsBatch(1, 4096, one, one, 4096, None, None, ctypes.cast(lens, ctypes.c_void_p))
    assert lib.ts_vote(ctypes.byref(c), ctypes.byref(beyond), one, 4096, one, None, one, one, None,
                       4096, None) == _lib.TS_EINVAL
    # table rows too short for a batch of 2
    short = _lib.TsBatch(2, 4096, one, one, 100, None)
    assert lib.ts_topk_ragged(ctypes.byref(c), ctypes.byref(short), one, 4096, None, None, one, one,
                              4096, one, one, 256, None) == _lib.TS_EINVAL
    # sel_stride below n_init + top_k + n_local
    assert lib.ts_topk_ragged(ctypes.byref(c), ctypes.byref(bt), one, 4096, None, None, one, one,
                              100, one, one, 256, None) == _lib.TS_EWORKSPACE
    # hit flags without a cache
    assert lib.ts_topk_ragged(ctypes.byref(c), ctypes.byref(bt), one, 4096, one, None, one, one,
                              4096, one, one, 256, None) == _lib.TS_EINVAL
    assert lib.ts_sparse_decode_attn(ctypes.byref(c), one, one, one, 10, one, 4096, one, 1, 2688,
                                     one, one, 16, None) == _lib.TS_EWORKSPACE
    assert lib.ts_paged_matmul(one, one, 10, one, one, 5, 10, 32, 8, 128, None) == _lib.TS_EINVAL
    assert lib.ts_paged_matmul(one, one, 10, one, one, 0, 10, 32, 8, 64, None) == _lib.TS_ESHAPE
    assert lib.ts_rope_apply(one, one, one, one, None, 1, 1, 4, 127, None) == _lib.TS_ESHAPE
    # pages of 16 tokens without a page pool
    assert lib.ts_kv_store(ctypes.byref(cfg(page_size=16)), one, one, one, None, one, one, 10, one, 100,
                           one, 1, 100, None) == _lib.TS_EINVAL
    assert "page pool" in err(lib)
    # more than 2^20 candidates per request
    huge = _lib.TsBatch(1, (1 << 20) + 641, one, one, 1 << 21, None)
    assert lib.ts_topk_ragged(ctypes.byref(c), ctypes.byref(huge), one, 1 << 21, None, None, one, one,
                              4096, one, one, 1 << 30, None) == _lib.TS_ESHAPE
    assert lib.ts_decode_layer(ctypes.byref(c), ctypes.byref(bt), one, one, one, one, one, 10, None,
                               one, one, one, 4096, one, one, 64, None) == _lib.TS_EWORKSPACE
    assert "workspace" in err(lib)


def test_misaligned_buffers_are_refused_on_the_host(lib):
    """Tensors are read with 16-byte vector loads and workspaces hold 8-byte atomics: a view at
    an odd offset fails the call instead of faulting the device."""
    c = cfg()
    one, odd = ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1004)
    bt = _lib.TsBatch(1, 4096, one, one, 4096, None)
    big = 1 << 30
    assert lib.ts_score_vote(ctypes.byref(c), ctypes.byref(bt), one, odd, 10, None, one, 4096, one, big,
                             None) == _lib.TS_EINVAL
    assert "k_pool must be aligned" in err(lib)
    assert lib.ts_score_vote(ctypes.byref(c), ctypes.byref(bt), one, one, 10, None, one, 4096,
                             ctypes.c_void_p(0x1010), big, None) == _lib.TS_EINVAL
    assert "workspace must be aligned to 256" in err(lib)
    assert lib.ts_topk_ragged(ctypes.byref(c), ctypes.byref(bt), one, 4096, None, None, one, one, 4096,
                              one, ctypes.c_void_p(0x1008), big, None) == _lib.TS_EINVAL
    assert lib.ts_sparse_decode_attn(ctypes.byref(c), odd, one, one, 10, one, 4096, one, 1, 2688,
                                     one, one, big, None) == _lib.TS_EINVAL
    assert "q must be aligned" in err(lib)
    # the stores and the projection: rows are copied as 16-byte vectors
    assert lib.ts_kv_store(ctypes.byref(c), one, odd, one, None, one, one, 10, one, 4096, one, 1, 4096,
                           None) == _lib.TS_EINVAL
    assert "v must be aligned" in err(lib)
    assert lib.ts_kv_store_chunk(ctypes.byref(c), one, one, one, None, 4, one, odd, 10, one, one, 4096,
                                 None) == _lib.TS_EINVAL
    assert "v_pool must be aligned" in err(lib)
    assert lib.ts_qkv_store(ctypes.byref(c), one, odd, None, 4096, one, None, one, one, one, 10, one,
                            4096, one, 1, 4096, None) == _lib.TS_EINVAL
    assert "w must be aligned" in err(lib)
    assert lib.ts_fingerprint(ctypes.byref(c), odd, 4, one, one, 4096, one, one) == _lib.TS_EINVAL
    assert "q must be aligned" in err(lib)


def test_static_scratch_entry_point_rejects_what_does_not_fit(lib):
    assert lib.ts_attn_static_scratch_bytes() == 4 << 20
    one = ctypes.c_void_p(0x1000)  # never dereferenced: the size check fails first
    wide = cfg(num_heads=64, num_kv_heads=8, top_k=4096)
    # 130 requests x 64 heads x 512 bytes of partials per head and split: above 4 MiB
    assert lib.ts_sparse_decode_attn_static(ctypes.byref(wide), one, one, one, 10, one, 4736, one,
                                            130, 4736, one, None) == _lib.TS_EWORKSPACE
    assert "scratch" in err(lib)
    assert lib.ts_sparse_decode_attn_static(ctypes.byref(cfg()), one, one, one, 10, None, 2688, one,
                                            1, 2688, one, None) == _lib.TS_EINVAL


def test_python_layer_refuses_cpu_tensors(lib):
    c = ops.LayerConfig(num_heads=4, num_kv_heads=2, n_init=1, n_local=2, top_k=4)
    x = torch.zeros(1, 4, 128, dtype=torch.bfloat16)
    t = torch.zeros(4, 128)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.rope_apply(x, t, t, None)
    bt = ops.Batch(torch.zeros(1, dtype=torch.int32), torch.zeros(1, 64, dtype=torch.int32), 64)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.score(c, bt, x, torch.zeros(64, 2, 128, dtype=torch.bfloat16))
    with pytest.raises(TypeError):
        ops.rope_apply(x.float(), t, t, None)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libtokenselect_hip.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        _lib.load()


def test_workspace_sizes_never_shrink_with_the_context_or_the_batch(lib):
    """A workspace sized for (batch, max_seq_len) must serve every smaller batch and every
    shorter context: the candidates per workgroup move in steps, so the sizes are taken
    from bounds that do not."""
    for heads, kv in ((32, 8), (28, 4), (8, 1)):
        c = cfg(num_heads=heads, num_kv_heads=kv)
        lens = list(range(700, 70000, 997)) + [32768, 32769, 131072, 131073, 262144, 262145, 1048576]
        for fn in (lib.ts_decode_layer_workspace_bytes, lib.ts_score_partials_bytes,
                   lib.ts_select_workspace_bytes, lib.ts_topk_workspace_bytes):
            sizes = [fn(ctypes.byref(c), 4, L) for L in sorted(lens)]
            assert all(x > 0 for x in sizes)
            assert sizes == sorted(sizes), fn.__name__
        by_batch = [lib.ts_decode_layer_workspace_bytes(ctypes.byref(c), B, 65536) for B in range(1, 33)]
        assert by_batch == sorted(by_batch)


def test_header_is_plain_c_and_agrees_with_the_ctypes_mirror(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 (no C++ in it), and a C program
    sees the struct sizes and field offsets that the ctypes mirror and the library use."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stddef.h>\n#include <stdio.h>\n#include "tokenselect.h"\n'
        'int main(void) {\n'
        '  printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(ts_config), sizeof(ts_batch), sizeof(ts_selcache),\n'
        '         offsetof(ts_batch, threshold_hint), offsetof(ts_batch, wait_us),\n'
        '         offsetof(ts_batch, workspace_clean), offsetof(ts_batch, host_seq_lens),\n'
        '         sizeof(ts_new_kv), offsetof(ts_new_kv, max_tokens));\n'
        '  return 0;\n}\n')
    exe = tmp_path / "layout"
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", include, str(src),
                    "-o", str(exe)], check=True)
    got = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    assert got == [ctypes.sizeof(_lib.TsConfig), ctypes.sizeof(_lib.TsBatch), ctypes.sizeof(_lib.TsSelCache),
                   _lib.TsBatch.threshold_hint.offset, _lib.TsBatch.wait_us.offset,
                   _lib.TsBatch.workspace_clean.offset, _lib.TsBatch.host_seq_lens.offset,
                   ctypes.sizeof(_lib.TsNewKv), _lib.TsNewKv.max_tokens.offset]
