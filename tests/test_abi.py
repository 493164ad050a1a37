"""CPU-only checks of the C ABI: the library loads, exports every symbol include/hyperattn.h declares,
the ctypes mirrors of its structs have the C layout, and argument errors are reported with a negative
status before anything is launched (so these calls are safe without a GPU)."""
import ctypes
import os
import re
import subprocess

import pytest

from hyperattention_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hyperattn.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return _lib.lib()


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ha_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    declared = _declared_symbols()
    assert declared == sorted(_lib.SYMBOLS)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in hyperattn.h but not exported"
    assert lib.ha_abi_version() == _lib.ABI_VERSION


def test_struct_layouts_match_the_header(tmp_path):
    """Compile a tiny C program against the header and compare sizeof/offsetof with ctypes."""
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "hyperattn.h"
int main(void) {
  printf("%zu %zu %zu\n", sizeof(ha_attn_operands), sizeof(ha_block_attn_args), sizeof(ha_forward_args));
  printf("%zu %zu %zu\n", offsetof(ha_attn_operands, scale), offsetof(ha_block_attn_args, accumulate),
         offsetof(ha_forward_args, workspace_bytes));
  printf("%zu %zu %zu\n", offsetof(ha_block_attn_args, q_idx), offsetof(ha_forward_args, scale),
         offsetof(ha_forward_args, v_stride_n));
  printf("%zu %zu %zu\n", sizeof(ha_attn_grads), offsetof(ha_attn_grads, workspace_bytes),
         offsetof(ha_attn_grads, accumulate));
  return 0;
}''')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    got = [int(x) for x in out]
    want = [ctypes.sizeof(_lib.AttnOperands), ctypes.sizeof(_lib.BlockAttnArgs), ctypes.sizeof(_lib.ForwardArgs),
            _lib.AttnOperands.scale.offset, _lib.BlockAttnArgs.accumulate.offset,
            _lib.ForwardArgs.workspace_bytes.offset, _lib.BlockAttnArgs.q_idx.offset, _lib.ForwardArgs.scale.offset,
            _lib.ForwardArgs.v_stride_n.offset,
            ctypes.sizeof(_lib.AttnGrads), _lib.AttnGrads.workspace_bytes.offset, _lib.AttnGrads.accumulate.offset]
    assert got == want


def test_argument_errors_before_any_launch(lib):
    one = ctypes.c_void_p(16)
    # null pointers
    assert lib.ha_lsh_hash(None, None, None, 1, 1, 128, 64, 8, 0, 0, 64, 0, 0, 0, None) == -1
    assert b"null" in lib.ha_last_error()
    # bad dtype, bad r, bad d
    assert lib.ha_lsh_hash(one, one, one, 1, 1, 128, 64, 8, 0, 0, 64, 0, 0, 7, None) == -2
    assert lib.ha_lsh_hash(one, one, one, 1, 1, 128, 64, 0, 0, 0, 64, 0, 0, 0, None) == -3
    assert b"Invalid value for num_projs" in lib.ha_last_error()
    assert lib.ha_lsh_hash(one, one, one, 1, 1, 128, 60, 8, 0, 0, 64, 0, 0, 0, None) == -4
    # sort: workspace too small, too many keys
    assert lib.ha_bucket_argsort_workspace_bytes(4, 8192, 256) == 4 * 2 * 256 * 4
    assert lib.ha_bucket_argsort(one, one, 0, 4, 8192, 8192, 0, 256, one, 16, None) == -6
    assert lib.ha_bucket_argsort(one, one, 0, 4, 8192, 8192, 0, 1 << 20, one, 1 << 30, None) == -5
    # the sort without a workspace: more scratch than the built-in array holds
    assert lib.ha_bucket_argsort_static(one, one, 0, 4096, 1 << 20, 1 << 20, 0, 256, None) == -6
    assert b"scratch" in lib.ha_last_error()
    assert lib.ha_bucket_argsort_static(one, one, 0, 0, 8, 8, 0, 256, None) == -3
    # gather: row bytes not a multiple of 16
    assert lib.ha_gather_rows(one, one, 0, one, 1, 1, 8, 8, 8, 3, 0, 0, 3, 2, None) == -4
    # merge
    assert lib.ha_lse_merge(one, one, one, one, one, one, 8, 12, 12, 12, 12, 1, 1, 1, 0, None) == -3
    two = ctypes.c_void_p(32)
    assert lib.ha_lse_merge(one, one, two, two, one, one, 8, 24, 24, 24, 24, 1, 1, 1, 0, None) == -5  # in place, d = 24
    assert b"in place" in lib.ha_last_error()
    assert lib.ha_lse_merge_segments(one, one, two, two, one, one, None, 2, 8, 24, 192, 24, 192, 24, 192, 24, 8, 8, 8, 8, 0, None) == -5
    assert lib.ha_lse_merge_segments(one, one, one, one, one, one, None, 2, 8, 12, 96, 12, 96, 12, 96, 12, 8, 8, 8, 8, 0, None) == -3
    assert lib.ha_lse_merge_segments(one, one, one, one, one, one, None, 2, 8, 16, 128, 16, 128, 16, 128, 16, 8, 8, 8, 8, 5, None) == -2
    assert lib.ha_lse_merge_segments(one, None, one, one, one, one, None, 2, 8, 16, 128, 16, 128, 16, 128, 16, 8, 8, 8, 8, 0, None) == -1


def _operands(**kw):
    t = _lib.AttnOperands()
    t.q = t.k = t.v = t.out = t.lse = 16
    t.batch, t.heads, t.n_q, t.n_k, t.d, t.dv = 1, 1, 256, 256, 64, 64
    t.q_stride_n = t.k_stride_n = t.v_stride_n = t.o_stride_n = 64
    t.segs, t.kv_group, t.scale, t.dtype = 1, 1, 0.125, 0
    for k, v in kw.items():
        setattr(t, k, v)
    return t


def test_attention_argument_errors(lib):
    assert lib.ha_flash_attn_fwd(None, 0, None) == -1
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(dtype=3)), 0, None) == -2
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(d=256, dv=256)), 0, None) == -4
    assert b"head dimensions up to 128" in lib.ha_last_error()
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(d=36, dv=36)), 0, None) == -5   # not a multiple of 8
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(d=64, dv=4)), 0, None) == -5
    assert b"multiples of 8" in lib.ha_last_error()
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(scale=0.0)), 0, None) == -3
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(q_stride_n=60)), 0, None) == -3
    # addressing limits: 2^24 rows, row strides below 16 MiB, one head within 4 GiB
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(n_k=1 << 24)), 0, None) == -3
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(k_stride_n=1 << 23)), 0, None) == -5
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(n_q=1 << 20, q_stride_n=4096)), 0, None) == -5
    assert b"4 GiB" in lib.ha_last_error()
    assert lib.ha_flash_attn_fwd(ctypes.byref(_operands(v_stride_n=-64)), 0, None) == -5
    a = _lib.BlockAttnArgs()
    a.t = _operands()
    a.q_idx = a.k_idx = 16
    a.q_idx_stride_n = a.k_idx_stride_n = 1
    a.block_size, a.sample_size = 256, 100
    assert lib.ha_block_attn_fwd(ctypes.byref(a), None) == -3  # sample_size % 128
    a.sample_size = 0
    a.t = _operands(n_k=192)
    assert lib.ha_block_attn_fwd(ctypes.byref(a), None) == -3
    assert b"divisible by 128" in lib.ha_last_error()
    a.t = _operands()
    a.k_idx_stride_n = 0
    assert lib.ha_block_attn_fwd(ctypes.byref(a), None) == -5
    a.k_idx_stride_n = 1
    a.q_idx = None
    assert lib.ha_block_attn_fwd(ctypes.byref(a), None) == -1


def test_forward_plan_and_workspace(lib):
    f = _lib.ForwardArgs()
    f.batch, f.heads, f.kv_heads, f.n, f.d, f.dv = 1, 32, 32, 131072, 64, 64
    f.lsh_num_projs, f.block_size, f.sample_size, f.min_seq_len = 8, 256, 256, 2048
    f.causal, f.scale, f.dtype = 1, 0.125, 0
    ws = lib.ha_forward_workspace_bytes(ctypes.byref(f))
    # byte-sized bucket ids of q and k (2 x 4 Mi) + per-unit orders (2 x 4 Mi x 4 B) + per-unit bucket counts
    # (2 x 32 sequences x 64 units of 2048 rows x 256 x 4 B) + six levels of (q_idx + k_idx) (2 x 2 Mi x 4 B each)
    assert ws == 2 * 4194304 + 2 * 4194304 * 4 + 2 * 32 * 64 * 1024 + 6 * 2 * 2097152 * 4
    f.lsh_num_projs = 12   # 4096 buckets: int32 ids, a sort per level with two digit passes and their orders in between
    ws12 = lib.ha_forward_workspace_bytes(ctypes.byref(f))
    assert ws12 > 2 * 4194304 * 4 + 3 * 6 * 2 * 2097152 * 4 and ws12 < 400 << 20
    f.lsh_num_projs = 17
    assert lib.ha_forward_workspace_bytes(ctypes.byref(f)) > 0   # sized; the call itself rejects more than 16 projections
    f.lsh_num_projs = 8
    f.n = 4096
    ws_even = lib.ha_forward_workspace_bytes(ctypes.byref(f))
    f.n = 4095  # an odd length: the hashed levels see the sequence with the appended zero row, 4096 rows
    assert lib.ha_forward_workspace_bytes(ctypes.byref(f)) == ws_even > 0
    f.n = 4097  # padded to 4098: halves of 2049 rows are hashed and must be a multiple of 128
    assert lib.ha_forward_workspace_bytes(ctypes.byref(f)) == -3
    f.n = 131072 + 2  # the first halves (65537) are hashed and must be a multiple of 128
    assert lib.ha_forward_workspace_bytes(ctypes.byref(f)) == -3
    f.n, f.min_seq_len, f.sample_size = 2048, 128, 256  # the deepest hashed level has 128 keys < 256 default samples
    assert lib.ha_forward_workspace_bytes(ctypes.byref(f)) == -3
    assert b"sampled rows" in lib.ha_last_error()
    f.min_seq_len = 2048
    f.n, f.causal = 4000, 0  # hashed path needs n % 128 == 0
    assert lib.ha_forward_workspace_bytes(ctypes.byref(f)) == -3
    f.n, f.min_seq_len = 1000, 2048  # exact path: no workspace needed beyond the minimum
    assert lib.ha_forward_workspace_bytes(ctypes.byref(f)) == 256
    assert lib.ha_forward(ctypes.byref(f), None) == -1  # null tensors
    # the first stage alone
    offs = (ctypes.c_int64 * 48)()
    levels = ctypes.c_int(0)
    assert lib.ha_forward_sort(None, offs, offs, ctypes.byref(levels), None) == -1
    assert lib.ha_forward_sort(ctypes.byref(f), offs, offs, ctypes.byref(levels), None) == -1  # null q, k
    f.q = f.k = 256
    f.d = 4
    assert lib.ha_forward_sort(ctypes.byref(f), offs, offs, ctypes.byref(levels), None) == -5
    f.d, f.n, f.min_seq_len, f.causal = 64, 1000, 2048, 1   # nothing hashed: no launch, no workspace needed
    assert lib.ha_forward_sort(ctypes.byref(f), offs, offs, ctypes.byref(levels), None) == 0 and levels.value == 0
    f.n, f.min_seq_len = 8192, 2048   # two hashed levels, but no workspace given
    assert lib.ha_forward_sort(ctypes.byref(f), offs, offs, ctypes.byref(levels), None) == -1  # null projection
    f.proj = 256
    assert lib.ha_forward_sort(ctypes.byref(f), offs, offs, ctypes.byref(levels), None) == -6
    assert levels.value == 2 and offs[0] > 0 and offs[1] > offs[0]


def test_merge_levels_argument_errors(lib):
    vp = ctypes.c_void_p
    one = vp(256)
    two = vp(512)
    arr = (vp * 1)(256)
    call = lambda levels, n, d, out=two, lse_out=two, dtype=0, o_un=arr: lib.ha_lse_merge_levels(
        one, one, o_un, arr, arr, one, out, lse_out, levels, 4, n, d, dtype, 0, None)
    assert lib.ha_lse_merge_levels(None, None, None, None, None, None, None, None, 0, 1, 128, 64, 0, 0, None) == -1
    assert call(1, 256, 64, dtype=3) == -2
    assert call(25, 1 << 25, 64) == -5            # more levels than the kernel is built for
    assert call(1, 256, 60) == -3                 # d % 8
    assert call(3, 1004, 64) == -3                # n not divisible by 2^levels
    assert call(1, 256, 64, out=one) == -5        # in place
    assert call(1, 256, 64, o_un=(vp * 1)(None)) == -1


def test_backward_argument_errors_before_any_launch(lib):
    t = _lib.AttnOperands()
    g = _lib.AttnGrads()
    assert lib.ha_flash_attn_bwd(None, 0, None, None) == -1
    assert lib.ha_flash_attn_bwd(ctypes.byref(t), 0, ctypes.byref(g), None) == -1  # null tensors
    assert lib.ha_attn_bwd_workspace_bytes(ctypes.byref(t), 0) == -3                # zero sizes
    t.batch, t.heads, t.n_q, t.n_k, t.d, t.dv, t.kv_group = 2, 4, 300, 200, 64, 64, 2
    assert lib.ha_attn_bwd_workspace_bytes(ctypes.byref(t), 0) == -3                # segs must be >= 1
    t.segs = 3   # three segments per head: three times the per-query and per-sample scratch
    assert lib.ha_attn_bwd_workspace_bytes(ctypes.byref(t), 0) == 3 * 19200
    assert lib.ha_attn_bwd_workspace_bytes(ctypes.byref(t), 128) == 3 * 19200 + 2 * 3 * 2 * 2 * 128 * 64 * 4
    t.segs = 1
    # two floats per query (256-byte aligned) + two fp32 (batch, kv_heads, sample_size, d) arrays
    assert lib.ha_attn_bwd_workspace_bytes(ctypes.byref(t), 0) == 19200
    assert lib.ha_attn_bwd_workspace_bytes(ctypes.byref(t), 128) == 19200 + 2 * (2 * 2 * 128 * 64 * 4)
    a = _lib.BlockAttnArgs()
    assert lib.ha_block_attn_bwd(ctypes.byref(a), ctypes.byref(g), None) == -1


def test_python_layer_fails_loudly_without_library(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "missing.so"))
    monkeypatch.setattr(_lib, "_lib", None)
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_sweep_script_command_line():
    """The sweep keeps the reference's options (benchmark_single_attention.py:14-22)."""
    from hyperattention_amd import benchmark_single_attention as sweep
    args = sweep.get_arguments(["--no_causal", "--smooth_block", "--mode", "fwd", "--attn_method", "hyper"])
    assert args.no_causal and args.smooth_block and args.mode == "fwd" and args.attn_method == "hyper"
    for mode in ("bwd", "fwd+bwd"):
        assert sweep.get_arguments(["--mode", mode]).mode == mode
    with pytest.raises(SystemExit):  # a CUDA-only package: stops before touching the GPU
        sweep.main(["--attn_method", "flash-cuda"])


def test_explicit_sample_lists_are_range_checked_on_the_host():
    """A sample list is local to the keys of each call; inside the causal recursion the shortest hashed
    level bounds it (a larger row number would name a key of the second half: a future token)."""
    import torch
    from hyperattention_amd import ops
    assert ops.smallest_hashed_key_length(8192, 1024, True) == 1024      # halves 4096, 2048, 1024
    assert ops.smallest_hashed_key_length(8192, 1025, True) == 2048      # 1024 < min_seq_len: exact there
    assert ops.smallest_hashed_key_length(8192, 4096, False) == 8192
    assert ops.smallest_hashed_key_length(1000, 4096, False) is None
    ok = torch.tensor([0, 5, 1023])
    ops.check_sampled_idx(ok, 1024)
    with pytest.raises(AssertionError, match="sampled_idx must lie in"):
        ops.check_sampled_idx(torch.tensor([0, 5, 1024]), 1024)
    with pytest.raises(AssertionError, match="sampled_idx must lie in"):
        ops.check_sampled_idx(torch.tensor([-1, 5]), 1024)
    ok[2] = 4000  # an in-place change is seen
    with pytest.raises(AssertionError):
        ops.check_sampled_idx(ok, 1024)
    # the argument block of one call checks against that call's key length
    q = torch.zeros((1, 256, 1, 64), dtype=torch.float16)
    idx = torch.zeros((1, 256, 1), dtype=torch.int32)
    lse = torch.zeros((1, 1, 256))
    with pytest.raises(AssertionError, match="sampled_idx must lie in"):
        ops._block_attn_args(q, q, q, q, lse, idx, idx, 128, 128, 0.125, False, torch.arange(200, 328))


def test_workspace_cache_policy():
    """The forward's workspace cache: one tensor per (device, stream) that only grows, a replaced tensor
    stays alive (a captured graph or queued work may point at it), a call under stream capture never shares
    or caches, and copies / pickles of a module start with an empty cache."""
    import copy
    import pickle
    import torch
    from hyperattention_amd import HyperAttention, ops
    c = ops.WorkspaceCache()
    cpu = torch.device("cpu")
    a = c.tensor(cpu, 0, 1000)
    assert a.numel() == 1000 and c.tensor(cpu, 0, 500) is a          # reused while it is large enough
    b = c.tensor(cpu, 0, 4000)
    assert b is not a and b.numel() == 4000 and any(t is a for t in c.retired)
    other_stream = c.tensor(cpu, 1, 100)
    assert other_stream is not b and c.tensor(cpu, 0, 100) is b      # one slot per stream
    g1, g2 = c.tensor(cpu, 0, 100, capturing=True), c.tensor(cpu, 0, 100, capturing=True)
    assert g1 is not g2 and g1 is not b and c.tensor(cpu, 0, 100) is b
    c.sizes[("shape",)] = 123
    for clone in (copy.deepcopy(c), pickle.loads(pickle.dumps(c))):
        assert clone.slots == {} and clone.sizes == {} and clone.retired == []
    m = HyperAttention(input_dim=64)
    m._workspace.tensor(cpu, 0, 64)
    m2 = copy.deepcopy(m)
    assert m2._workspace.slots == {} and torch.equal(m2.lsh.proj_dir, m.lsh.proj_dir)
    import io
    buf = io.BytesIO()
    torch.save(m, buf)
    assert len(buf.getvalue()) < 100000


def test_sampled_idx_bounds_of_an_inference_tensor():
    """A sample list created under inference mode has no version counter: it is checked without one."""
    import torch
    from hyperattention_amd import ops
    with torch.inference_mode():
        idx = torch.arange(0, 128)
    ops.check_sampled_idx(idx, 128)
    with pytest.raises(AssertionError, match="sampled_idx must lie in"):
        ops.check_sampled_idx(idx, 100)
    assert not hasattr(idx, "_ha_bounds")
