"""JIT boundary without a GPU: generated source, cache layout, compile (hipcc cross-compiles gfx950), exported
symbol, argument checking and failure modes. Restates what can be checked of the reference's
tests/test_jit.py:31-64 and of yan/jit/{template,compiler,runtime}.py on a machine with no device."""
import ctypes
import os
import subprocess

import pytest
import torch

from yan_amd import jit
from yan_amd.jit import compiler, runtime, template

ARGS = (('lhs', torch.float8_e4m3fn), ('rhs', torch.float8_e4m3fn), ('scale', torch.float), ('out', torch.bfloat16),
        ('enable_double_streams', bool), ('stream', torch.cuda.Stream))


@pytest.fixture()
def cache_dir(tmp_path, monkeypatch):
    monkeypatch.setenv('YAN_CACHE_DIR', str(tmp_path))
    saved = compiler.runtime_cache.cache
    compiler.runtime_cache.cache = {}
    yield tmp_path
    compiler.runtime_cache.cache = saved


def test_cpp_format_leaves_cpp_braces_alone():
    src = 'constexpr auto N = {N}; struct S { int x{K}; }; // {UNKNOWN} {N}'
    assert jit.cpp_format(src, {'N': 7168, 'K': 3}) == 'constexpr auto N = 7168; struct S { int x3; }; // {UNKNOWN} 7168'


def test_generate_signature_and_casts():
    code = jit.generate(('"gemm/utils.hpp"', '<vector>'), ARGS, '\nint x = 1;\n')
    sig = ('extern "C" EXPORT_API void launch(void* __raw_lhs, void* __raw_rhs, void* __raw_scale, void* __raw_out, '
           'bool enable_double_streams, void* __raw_stream, int& __return_code) {')
    assert sig in code
    assert 'auto lhs = reinterpret_cast<__hip_fp8_e4m3*>(__raw_lhs);' in code
    assert 'auto scale = reinterpret_cast<float*>(__raw_scale);' in code
    assert 'auto out = reinterpret_cast<__hip_bfloat16*>(__raw_out);' in code
    assert 'auto stream = reinterpret_cast<hipStream_t>(__raw_stream);' in code
    assert 'enable_double_streams = ' not in code            # scalars cross by value, no cast
    assert '#include <hip/hip_runtime.h>' in code and '#include <vector>' in code and '#include "gemm/utils.hpp"' in code
    assert code.index('#include <vector>') < code.index('#include "gemm/utils.hpp"') < code.index('extern "C"')
    assert '    int x = 1;' in code and code.rstrip().endswith('}')
    assert 'cuda' not in code.lower()


def test_type_maps_cover_the_reference_surface():
    for t in (bool, int, float, torch.int, torch.float, torch.half, torch.bfloat16, torch.float8_e4m3fn, torch.cuda.Stream):
        assert t in template.typename_map and t in template.ctype_map and t in template.genc_map
    assert template.typename_map[torch.half] == 'torch.half' and template.typename_map[int] == 'int'
    assert template.ctype_map[int] is ctypes.c_int and template.ctype_map[torch.bfloat16] is ctypes.c_void_p
    t = torch.zeros(4, dtype=torch.bfloat16)
    assert template.map_ctype(t).value == t.data_ptr()
    assert template.map_ctype(3).value == 3 and template.map_ctype(True).value is True
    assert template.map_ctype(0.5).value == 0.5


def test_compiler_discovery():
    path, version = jit.get_hipcc_compiler()
    assert os.path.exists(path) and tuple(int(x) for x in version.split('.')) >= (6, 4)
    assert jit.get_nvcc_compiler() == (path, version)          # the name callers of the reference use


def test_build_layout_cache_and_export(cache_dir):
    body = '\nstd::cout << enable_double_streams << std::endl;\n__return_code = 7;\n'
    code = jit.generate((), ARGS, body)
    rt = jit.build('test_func', ARGS, code)
    name = os.path.basename(rt.path)
    assert name.startswith('kernel.test_func.') and len(name.split('.')[-1]) == 12
    assert os.path.dirname(rt.path) == str(cache_dir / 'cache')
    assert sorted(os.listdir(rt.path)) == ['kernel.args', 'kernel.cu', 'kernel.so']
    assert open(os.path.join(rt.path, 'kernel.cu')).read() == code
    assert open(os.path.join(rt.path, 'kernel.args')).read() == (
        "('lhs', torch.float8_e4m3fn), ('rhs', torch.float8_e4m3fn), ('scale', torch.float), ('out', torch.bfloat16), "
        "('enable_double_streams', bool), ('stream', torch.cuda.Stream)")
    assert os.listdir(cache_dir / 'tmp') == []                 # temporaries were renamed into place
    # exactly one entry point, with C linkage
    lib = ctypes.CDLL(os.path.join(rt.path, 'kernel.so'))
    assert hasattr(lib, 'launch')
    syms = subprocess.check_output(['nm', '-D', '--defined-only', os.path.join(rt.path, 'kernel.so')], text=True)
    assert [ln.split()[-1] for ln in syms.splitlines() if ' T ' in ln] == ['launch']
    # same (name, code) -> the same object from memory; a fresh process-level cache finds it on disk
    assert jit.build('test_func', ARGS, code) is rt
    mtime = os.path.getmtime(os.path.join(rt.path, 'kernel.so'))
    compiler.runtime_cache.cache = {}
    again = jit.build('test_func', ARGS, code)
    assert again.path == rt.path and os.path.getmtime(os.path.join(rt.path, 'kernel.so')) == mtime
    # different code or name -> different directory
    assert jit.build('test_func', ARGS, jit.generate((), ARGS, body + '\n')).path != rt.path
    assert compiler.kernel_dir('other', code) != compiler.kernel_dir('test_func', code)
    # the code object really is gfx950
    objs = subprocess.run(['/opt/rocm/llvm/bin/clang-offload-bundler', '--list', '--type=o',
                           f'--input={os.path.join(rt.path, "kernel.so")}'], capture_output=True, text=True)
    if objs.returncode == 0 and objs.stdout.strip():
        assert 'gfx950' in objs.stdout


def test_concurrent_builds_of_one_kernel_leave_one_valid_entry(cache_dir):
    """Several processes that miss the cache at the same moment each compile into a temporary of their own and rename
    it into place (yan/jit/compiler.py:131-151, 228-250 does the same): all succeed, one directory remains, and it
    loads."""
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prog = ("import sys, torch; sys.path.insert(0, %r); from yan_amd import jit; "
            "args = (('x', torch.float), ('n', int)); "
            "rt = jit.build('racer', args, jit.generate((), args, '\\n__return_code = n + 1;\\n')); print(rt.path)") % root
    env = dict(os.environ, YAN_CACHE_DIR=str(cache_dir))
    procs = [subprocess.Popen([sys.executable, '-c', prog], env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
             for _ in range(3)]
    outs = [p.communicate(timeout=300) for p in procs]
    assert all(p.returncode == 0 for p in procs), [e[-500:] for _, e in outs]
    paths = {o.strip().splitlines()[-1] for o, _ in outs}
    assert len(paths) == 1
    path = paths.pop()
    assert os.listdir(cache_dir / 'cache') == [os.path.basename(path)]
    assert sorted(os.listdir(path)) == ['kernel.args', 'kernel.cu', 'kernel.so']
    assert os.listdir(cache_dir / 'tmp') == []
    assert hasattr(ctypes.CDLL(os.path.join(path, 'kernel.so')), 'launch')


def test_runtime_call_marshals_and_checks_arguments(cache_dir):
    # a host-only body: the launch wrapper itself needs no device
    args = (('n', int), ('x', float), ('flag', bool), ('data', torch.int))
    body = '\n__return_code = n + (flag ? 100 : 0) + static_cast<int>(x * 10) + (data != nullptr ? 1000 : 0);\n'
    rt = jit.build('host_only', args, jit.generate((), args, body))
    data = torch.zeros(4, dtype=torch.int)
    assert rt(5, 0.5, True, data) == 5 + 100 + 5 + 1000
    assert rt(1, 0.0, False, data) == 1001
    with pytest.raises(AssertionError, match='Expected 4 arguments'):
        rt(5, 0.5, True)
    with pytest.raises(AssertionError, match='dtype'):
        rt(5, 0.5, True, torch.zeros(4, dtype=torch.float))
    with pytest.raises(AssertionError, match='built-in type'):
        rt(5.0, 0.5, True, data)


def test_compile_failure_raises_runtime_error(cache_dir):
    args = (('n', int),)
    with pytest.raises(RuntimeError, match='Failed to compile'):
        jit.build('broken', args, jit.generate((), args, '\nthis is not C++;\n'))
    # an unreplaced template key is a compile error too, not a silent default
    with pytest.raises(RuntimeError, match='Failed to compile'):
        jit.build('unkeyed', args, jit.generate((), args, jit.cpp_format('\nconstexpr int B = {BLOCK_M};\n', {})))


def test_incomplete_cache_directory_is_rebuilt(cache_dir):
    args = (('n', int),)
    code = jit.generate((), args, '\n__return_code = n * 2;\n')
    rt = jit.build('rebuild', args, code)
    os.unlink(os.path.join(rt.path, 'kernel.so'))
    assert not runtime.Runtime.is_path_valid(rt.path)
    compiler.runtime_cache.cache = {}
    again = jit.build('rebuild', args, code)
    assert runtime.Runtime.is_path_valid(again.path) and again(21) == 42
    with pytest.raises(AssertionError):
        runtime.Runtime(str(cache_dir / 'nowhere'))


def test_header_digest_tracks_header_contents():
    v = compiler.get_yan_version()
    assert len(v) == 12 and v == compiler.get_yan_version()
    assert os.path.isdir(os.path.join(compiler.get_jit_include_dir(), 'gemm'))


def test_gemm_kernels_compile_for_gfx950(cache_dir):
    """The two GEMM translation units the op layer generates build without a device (smallest tiles)."""
    from yan_amd.jit_kernels import bf16_gemm, gemm
    name, keys, defs = bf16_gemm.dense_kernel_plan(64, 64, 64, torch.bfloat16, 256)
    rt = jit.build(name, defs, jit.generate(bf16_gemm.includes, defs, jit.cpp_format(bf16_gemm.template, keys)))
    assert runtime.Runtime.is_path_valid(rt.path)
    name, keys, defs, _, tmpl = gemm.fp8_kernel_plan(1, 128, 128, 256)
    rt = jit.build(name, defs, jit.generate(gemm.includes, defs, jit.cpp_format(tmpl, keys)))
    assert runtime.Runtime.is_path_valid(rt.path)
