"""Host-side behaviour of the façade that needs no GPU."""
import pytest
import torch

import rwkv_ops_amd
from rwkv_ops_amd.synthetic import make_inputs


def test_facade_names():
    fn, use_kernel = rwkv_ops_amd.get_generalized_delta_rule(64, "hip")
    assert use_kernel is True and fn is rwkv_ops_amd.generalized_delta_rule
    assert rwkv_ops_amd.rwkv7_op is rwkv_ops_amd.generalized_delta_rule
    assert rwkv_ops_amd.RWKV7_USE_KERNEL is True
    assert rwkv_ops_amd.get_generalized_delta_rule(KERNEL_TYPE="triton")[1] is True
    assert rwkv_ops_amd.get_generalized_delta_rule(128)[0] is rwkv_ops_amd.generalized_delta_rule
    with pytest.raises(NotImplementedError):
        rwkv_ops_amd.get_generalized_delta_rule(256)
    with pytest.raises(NotImplementedError):
        rwkv_ops_amd.get_generalized_delta_rule(64, "native")


def test_no_cpu_fallback():
    r, w, k, v, a, b, h0 = make_inputs(1, 4, 2, 64, seed=0)
    with pytest.raises(RuntimeError, match="MI355X"):
        rwkv_ops_amd.generalized_delta_rule(r, w, k, v, a, b, h0)


def test_shape_validation_happens_first():
    r, w, k, v, a, b, h0 = make_inputs(1, 4, 2, 64, seed=0)
    with pytest.raises(ValueError):
        rwkv_ops_amd.generalized_delta_rule(r, w[:, :2], k, v, a, b)
    with pytest.raises(ValueError):
        rwkv_ops_amd.generalized_delta_rule(r[0], w[0], k[0], v[0], a[0], b[0])


def test_product_does_not_import_oracle():
    import os
    root = os.path.dirname(os.path.abspath(rwkv_ops_amd.__file__))
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f


def test_state_map_needs_initial_state():
    r, w, k, v, a, b, _ = make_inputs(2, 4, 2, 64, seed=0)
    with pytest.raises(ValueError, match="state_map"):
        rwkv_ops_amd.generalized_delta_rule(r, w, k, v, a, b, state_map=[0, 1])


def test_cu_seqlens_checks_follow_the_reference():
    """The checks of chunk_dplr_delta_rule (torch_op.py:388-398), raised before anything touches a device."""
    r, w, k, v, a, b, h0 = make_inputs(2, 8, 2, 64, seed=0)
    with pytest.raises(ValueError, match="batch size is expected to be 1 rather than 2"):
        rwkv_ops_amd.generalized_delta_rule(r, w, k, v, a, b, cu_seqlens=[0, 3, 8])
    one = [x[:1] for x in (r, w, k, v, a, b)]
    with pytest.raises(ValueError, match="number of initial states is expected to be equal to the number of input "
                                         "sequences, i.e., 3 rather than 2"):
        rwkv_ops_amd.generalized_delta_rule(*one, initial_state=h0, cu_seqlens=[0, 3, 5, 8])
    with pytest.raises(ValueError, match="head_first"):
        rwkv_ops_amd.generalized_delta_rule(*one, head_first=True, cu_seqlens=[0, 3, 8])
    with pytest.raises(ValueError, match="state_map"):
        rwkv_ops_amd.generalized_delta_rule(*one, initial_state=h0, state_map=[0], cu_seqlens=[0, 8])
    with pytest.raises(RuntimeError, match="MI355X"):        # well-formed: only the device is missing
        rwkv_ops_amd.generalized_delta_rule(*one, initial_state=h0, cu_seqlens=[0, 3, 8])


def test_cu_seqlens_table_checks():
    from rwkv_ops_amd.rwkv7.op import _as_cu_seqlens
    dev = torch.device("cpu")
    assert _as_cu_seqlens([0, 3, 8], 8, dev).dtype == torch.int32
    assert _as_cu_seqlens(torch.tensor([0, 3, 3, 6]), 8, dev).tolist() == [0, 3, 3, 6]
    for bad in ([1, 3, 8], [0, 5, 3, 8], [0, 3, 9], [0], [[0, 3]]):
        with pytest.raises(ValueError):
            _as_cu_seqlens(bad, 8, dev)
    with pytest.raises(ValueError):
        _as_cu_seqlens(torch.tensor([0.0, 8.0]), 8, dev)


def test_custom_ops_have_shape_functions():
    """The torch.library ops trace without a device (what torch.compile needs): output shapes and dtypes."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    ops = torch.ops.rwkv_ops_amd
    with FakeTensorMode():
        B, T, H = 2, 100, 3
        xs = [torch.empty(B, T, H, 64, dtype=torch.bfloat16, device="cuda") for _ in range(6)]
        h0 = torch.empty(B, H, 64, 64, device="cuda")
        o, s = ops.rwkv7_fwd(*xs, h0, True, None)
        assert o.shape == xs[0].shape and o.dtype == torch.bfloat16
        assert tuple(s.shape) == (B, H, 64, 64) and s.dtype == torch.float32
        o, s = ops.rwkv7_fwd(*xs, None, False, None)
        assert s.numel() == 0
        grads = ops.rwkv7_bwd(*xs, h0, xs[0], h0)
        assert [tuple(g.shape) for g in grads] == [tuple(xs[0].shape)] * 6 + [(B, H, 64, 64)]
        cu = torch.empty(5, dtype=torch.int32, device="cuda")
        packed = [torch.empty(1, T, H, 64, dtype=torch.bfloat16, device="cuda") for _ in range(6)]
        o, s = ops.rwkv7_fwd_varlen(*packed, None, True, cu)
        assert o.shape == packed[0].shape and tuple(s.shape) == (4, H, 64, 64)
        grads = ops.rwkv7_bwd_varlen(*packed, None, None, None, cu)
        assert tuple(grads[6].shape) == (4, H, 64, 64) and grads[0].shape == packed[0].shape
        step = [torch.empty(B, H, 64, dtype=torch.bfloat16, device="cuda") for _ in range(6)]
        assert ops.rwkv7_decode(*step, h0).shape == step[0].shape
        pool = torch.empty(7, H, 64, 64, device="cuda")
        assert ops.rwkv7_decode_pool(*step, pool, torch.empty(B, dtype=torch.int32, device="cuda")).shape == step[0].shape


def test_forward_calls_look_at_the_giveup_word():
    """Both forward implementations call ``_lib.raise_if_gave_up`` before they launch (the GPU test sets the word)."""
    import inspect
    from rwkv_ops_amd.rwkv7 import op
    for fn in (op._fwd_impl, op._fwd_varlen_impl):
        assert "raise_if_gave_up" in inspect.getsource(fn)


def test_backward_clamps_a_state_map():
    """The autograd backward gathers and scatters through a clamped copy of the map (a device map is never checked)."""
    import inspect
    from rwkv_ops_amd.rwkv7 import op
    src = inspect.getsource(op._fwd_backward)
    assert "clamp_(0, h0_arg.shape[0] - 1)" in src and "index_add_(0, rows" in src
