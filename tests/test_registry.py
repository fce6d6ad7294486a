"""Behaviour tables of the registry boundary (CPU): matching, selection, caching, registration rules.

Restated from dlblas/op_registry.py:32-136, dlblas/op_struct.py:14-161, dlblas/cache.py:63-75 and the reference's
own tests (tests/test_registry.py:10-15, tests/test_cache.py:10-68, tests/test_symbolic_var.py:9-45)."""
import pytest
import torch

import dlblas_amd
from dlblas_amd.cache import Cache
from dlblas_amd.op_registry import OpRegistry, op_registry
from dlblas_amd.op_struct import OpImpl, OpParams, match, parse_args, violate_symbolic_constraints
from dlblas_amd.symbolic_var import SymVar, Tensor
from dlblas_amd.utils import get_args_from_op_name, get_list_op_names, get_op, register_dlblas_op


def _cpu_args(dtype=torch.float32):
    m, n, k = SymVar('m'), SymVar('n'), SymVar('k')
    return (Tensor((m, k), dtype=dtype, device='cpu'), Tensor((k, n), dtype=dtype, device='cpu'))


def test_fp8_ops_are_registered_at_import():
    names = get_list_op_names()
    for name in ('fp8_gemm', 'fp8_gemm_grouped_contiguous', 'fp8_gemm_grouped_masked', 'per_token_group_quant_fp8'):
        assert name in names
    both = get_args_from_op_name('fp8_gemm')   # two implementations under one name, identical parameter lists
    assert len(both) == 2 and both[0] == both[1]
    params = both[0]
    assert params.n_args == 4 and params.args_types == ['tensor'] * 4
    assert [a.dtype for a in params.args] == [torch.float8_e4m3fn] * 2 + [torch.float32] * 2
    assert all(a.device == 'cuda' for a in params.args)


def test_registration_is_idempotent_per_call():
    from dlblas_amd.kernels import fp8_gemm as mod
    before = op_registry.get_op_count('fp8_gemm')
    mod._register()
    assert op_registry.get_op_count('fp8_gemm') == before


def test_unknown_op_and_bad_args():
    with pytest.raises(NameError):
        get_op('no_such_op', (torch.zeros(1), ))
    with pytest.raises(TypeError):
        match([torch.zeros(1)], parse_args(_cpu_args()))
    with pytest.raises(TypeError):
        match((torch.zeros(1), ), 'not params')
    with pytest.raises(TypeError):
        parse_args((1.5, ))


def test_no_candidate_raises_lookup_error_on_cpu_tensors():
    a = torch.zeros(4, 128).to(torch.float8_e4m3fn)
    with pytest.raises(LookupError):  # registered for 'cuda' devices only
        get_op('fp8_gemm', (a, a, torch.zeros(4, 1), torch.zeros(1, 1)))


def test_parse_args_kind_tags():
    p = parse_args((Tensor((SymVar('m'), ), dtype=torch.float32, device='cpu'), 'relu', 3, torch.SymInt, torch.SymFloat,
                    torch.SymBool))
    assert p.args_types == ['tensor', 'str', 'int', 'int', torch.SymFloat, torch.SymBool]


def test_params_equality_ignores_dtype_device_shape():
    a = parse_args(_cpu_args(torch.float32))
    b = parse_args((Tensor((SymVar('x'), ), dtype=torch.float16, device='cuda'),
                    Tensor((SymVar('y'), SymVar('z'), SymVar('w')), dtype=torch.int8, device='cuda')))
    assert a == b
    assert not (a == parse_args(_cpu_args() + ('act', )))
    assert not (a == parse_args((_cpu_args()[0], 'act')))


def test_match_truth_table():
    params = parse_args(_cpu_args() + ('act', 7, torch.SymFloat, torch.SymBool))
    a, b = torch.zeros(3, 5), torch.zeros(5, 2)
    assert match((a, b, 'x', 1, 0.5, True), params)
    assert match((a, None, 'x', 1, 0.5, True), params), 'None skips every check'
    assert not match((a, b, 'x', 1, 0.5), params), 'arity'
    assert not match((a, b, 3, 1, 0.5, True), params), 'str expected'
    assert not match((a, b, 'x', 'y', 0.5, True), params), 'int expected'
    assert not match((a, b, 'x', 1, 1, True), params), 'float expected'
    assert not match((a, b, 'x', 1, 0.5, 1), params), 'bool expected'
    assert not match((a, 5, 'x', 1, 0.5, True), params), 'tensor expected'
    assert not match((a.half(), b, 'x', 1, 0.5, True), params), 'dtype'
    assert not match((a, torch.zeros(4, 2), 'x', 1, 0.5, True), params), 'k bound to 5 and 4'
    assert not match((a, torch.zeros(5), 'x', 1, 0.5, True), params), 'missing dim'
    cuda_params = parse_args((Tensor((SymVar('m'), ), dtype=torch.float32, device='cuda'), ))
    assert not match((torch.zeros(3), ), cuda_params), 'device prefix'


def test_violate_symbolic_constraints_table():
    sm, sn, sk = SymVar('m'), SymVar('n'), SymVar('k')
    assert not violate_symbolic_constraints([(1, 3), (3, 2)], [(sm, sk), (sk, sn)])
    assert violate_symbolic_constraints([(1, 3), (4, 2)], [(sm, sk), (sk, sn)])
    assert violate_symbolic_constraints([(1, ), (3, 2)], [(sm, sk), (sk, sn)])
    assert SymVar('m') == SymVar('m') and SymVar('m') != SymVar('n') and hash(SymVar('m')) == hash(SymVar('m'))
    assert SymVar('m') != 'm'


def test_selection_benches_every_candidate_and_caches_the_fastest():
    reg = OpRegistry()
    calls = []

    def make(tag, ms):
        def call(a, b):
            return tag

        def bench(a, b):
            calls.append(tag)
            return ms

        return call, bench

    for tag, ms in (('slow', 3.0), ('fast', 1.0), ('mid', 2.0)):
        call, bench = make(tag, ms)
        reg.register('mm', None, _cpu_args(), call, bench, call)
    call16, bench16 = make('half', 0.1)
    reg.register('mm', None, _cpu_args(torch.float16), call16, bench16, call16)
    a, b = torch.zeros(3, 5), torch.zeros(5, 2)
    op = reg.get_op('mm', (a, b))
    assert isinstance(op, OpImpl) and op(a, b) == 'fast'
    assert calls == ['slow', 'fast', 'mid'], 'the fp16 implementation does not match fp32 tensors'
    assert reg.get_op('mm', (a, b)) is op and calls == ['slow', 'fast', 'mid'], 'second lookup is a cache hit'
    assert reg.get_op('mm', (torch.zeros(4, 5), b))(a, b) == 'fast' and len(calls) == 6, 'new shape, new key'
    assert reg.get_op('mm', (a.half(), b.half()))(a, b) == 'half'
    # a single candidate is still benched (dlblas/op_registry.py:130-135)
    assert calls[-1] == 'half'


def test_explicit_cache_key():
    reg = OpRegistry()
    benched = []
    reg.register('f', None, _cpu_args(), lambda a, b: 1, lambda a, b: benched.append(1) or 1.0, None)
    a, b = torch.zeros(3, 5), torch.zeros(5, 2)
    op = reg.get_op('f', (a, b), cache_key='f_cols=5')
    assert reg.get_op('f', (torch.zeros(9, 5), b), cache_key='f_cols=5') is op and len(benched) == 1


def test_same_name_needs_same_signature():
    reg = OpRegistry()
    reg.register('g', None, _cpu_args(), lambda a, b: 0, lambda a, b: 1.0, None)
    with pytest.raises(AssertionError, match='must have the same parameters'):
        reg.register('g', None, _cpu_args() + ('act', ), lambda a, b, c: 0, lambda a, b, c: 1.0, None)


def test_cache_key_format_and_fp8_dtype():
    cache = Cache()
    a = torch.zeros(1, 2, dtype=torch.float16)
    b = torch.zeros(2, 1, dtype=torch.float16)
    assert cache.gen_key('matmul', (a, b, 'leaky_relu')) == 'matmul-0:f16_1x2-1:f16_2x1-2:leaky_relu'
    f8 = torch.zeros(4, 128).to(torch.float8_e4m3fn)
    assert cache.gen_key('fp8_gemm', (f8, torch.zeros(4, 1))) == 'fp8_gemm-0:f8e4m3_4x128-1:f32_4x1'
    with pytest.raises(LookupError):
        cache.gen_key('x', (torch.zeros(1, dtype=torch.complex64), ))


def test_cache_round_trips_through_a_file(tmp_path):
    reg = OpRegistry()
    reg.register('h', None, _cpu_args(), lambda a, b: 'one', lambda a, b: 2.0, None)
    reg.register('h', None, _cpu_args(), lambda a, b: 'two', lambda a, b: 1.0, None)
    a, b = torch.zeros(3, 5), torch.zeros(5, 2)
    best = reg.get_op('h', (a, b))
    reg.cache.to_file(str(tmp_path / 'sel'))
    fresh = Cache()
    fresh.from_file(str(tmp_path / 'sel'), reg.ops)
    assert fresh.get('h', (a, b), None) is best


def test_compat_aliases():
    import sys

    from dlblas_amd import compat
    saved = {k: sys.modules.get(k) for k in list(compat._ALIASES) + ['deep_gemm', 'dlblas.layers', 'dlblas.layers.moe', 'dlblas.layers.moe.kernels']}
    try:
        compat.install()
        from dlblas.kernels.fp8_gemm import fp8_gemm
        from dlblas.utils import get_op as g2
        import deep_gemm
        assert fp8_gemm is dlblas_amd.fp8_gemm and g2 is get_op
        for name in ('m_grouped_fp8_gemm_nt_contiguous', 'm_grouped_fp8_gemm_nt_masked',
                     'm_grouped_gemm_fp8_fp8_bf16_nt_contiguous', 'm_grouped_gemm_fp8_fp8_bf16_nt_masked'):
            assert hasattr(deep_gemm, name)
        assert deep_gemm.ceil_div(5, 4) == 2
        from dlblas.kernels.moe import silu_and_mul_masked_post_quant_fwd
        from dlblas.layers.moe.kernels.activation import silu_and_mul
        from dlblas_amd.kernels import activation as act_mod, moe as moe_mod
        assert silu_and_mul is act_mod.silu_and_mul
        assert silu_and_mul_masked_post_quant_fwd is moe_mod.silu_and_mul_masked_post_quant_fwd
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def test_argument_validation_happens_before_any_gpu_work():
    from dlblas_amd.kernels.fp8_gemm import fp8_gemm
    from dlblas_amd.kernels.fp8_gemm_grouped import fp8_gemm_grouped_contiguous
    a = torch.zeros(8, 256).to(torch.float8_e4m3fn)
    b = torch.zeros(128, 256).to(torch.float8_e4m3fn)
    with pytest.raises(AssertionError, match='Input tensors must be contiguous'):
        fp8_gemm(a[:, ::2], b, torch.zeros(8, 2), torch.zeros(1, 2))
    with pytest.raises(AssertionError, match='Scaling factor tensors must be contiguous'):
        fp8_gemm(a, b, torch.zeros(8, 4)[:, ::2], torch.zeros(1, 2))
    with pytest.raises(TypeError):
        fp8_gemm(a.float(), b, torch.zeros(8, 2), torch.zeros(1, 2))
    with pytest.raises(ValueError):
        fp8_gemm(a, b, torch.zeros(8, 3), torch.zeros(1, 2))
    with pytest.raises(ValueError):
        fp8_gemm_grouped_contiguous(a, torch.zeros(8, 2), b.reshape(1, 128, 256), torch.zeros(1, 1, 2),
                                    torch.zeros(8, 64, dtype=torch.bfloat16), torch.zeros(8, dtype=torch.int32))
