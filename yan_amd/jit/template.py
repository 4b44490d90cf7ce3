"""Source generation for JIT kernels: type registry, `{KEY}` substitution and the `launch` wrapper.

Mirrors the contract of the reference's `yan/jit/template.py` (type maps :12-58, `cpp_format` :61-66,
`generate` :69-154): every JIT kernel is one translation unit that exports a single
`extern "C" void launch(<one parameter per arg_def>, int& __return_code)`; tensors and streams cross the
boundary as `void* __raw_<name>` and are re-typed inside the wrapper, scalars cross by value.
The generated code is HIP for gfx950, there is no CUDA spelling anywhere.
"""
import ctypes
import os
from dataclasses import dataclass
from typing import Any, Dict, Iterable, Tuple

import torch


@dataclass(frozen=True)
class ArgKind:
    """One row of the boundary's type table."""
    py_name: str      # spelling used in `kernel.args` (evaluated back with `torch` in scope)
    ctype: Any        # ctypes class used to marshal the value
    abi_type: str     # C type in the `launch` parameter list
    typed: str        # C type the body sees (differs from abi_type => a cast is emitted)


_KINDS: Dict[Any, ArgKind] = {
    bool: ArgKind('bool', ctypes.c_bool, 'bool', 'bool'),
    int: ArgKind('int', ctypes.c_int, 'int', 'int'),
    float: ArgKind('float', ctypes.c_float, 'float', 'float'),
    torch.int: ArgKind('torch.int', ctypes.c_void_p, 'void*', 'int*'),
    torch.uint8: ArgKind('torch.uint8', ctypes.c_void_p, 'void*', 'uint8_t*'),      # raw device bytes (workspaces)
    torch.float: ArgKind('torch.float', ctypes.c_void_p, 'void*', 'float*'),
    torch.float16: ArgKind('torch.half', ctypes.c_void_p, 'void*', '__half*'),
    torch.bfloat16: ArgKind('torch.bfloat16', ctypes.c_void_p, 'void*', '__hip_bfloat16*'),
    # OCP e4m3 (max 448, no inf): the format gfx950's MFMA consumes; kernels treat it as raw bytes.
    torch.float8_e4m3fn: ArgKind('torch.float8_e4m3fn', ctypes.c_void_p, 'void*', '__hip_fp8_e4m3*'),
    torch.cuda.Stream: ArgKind('torch.cuda.Stream', ctypes.c_void_p, 'void*', 'hipStream_t'),
}

# The three dict views the reference exposes under these names (template.py:12-49).
typename_map: Dict[Any, str] = {t: k.py_name for t, k in _KINDS.items()}
ctype_map: Dict[Any, Any] = {t: k.ctype for t, k in _KINDS.items()}
genc_map: Dict[Any, Tuple[str, str]] = {t: (k.abi_type, k.typed) for t, k in _KINDS.items()}

_SYS_INCLUDES = ('<hip/hip_runtime.h>', '<hip/hip_bf16.h>', '<hip/hip_fp16.h>', '<hip/hip_fp8.h>',
                 '<cstdint>', '<iostream>')
_RAW = '__raw_'


def map_ctype(value: Any) -> Any:
    """Python value -> ctypes value for one `launch` argument (reference: template.py:52-58)."""
    if isinstance(value, torch.Tensor):
        return _KINDS[value.dtype].ctype(value.data_ptr())
    if isinstance(value, torch.cuda.Stream):
        # On ROCm `cuda_stream` is the hipStream_t handle.
        return ctypes.c_void_p(value.cuda_stream)
    return _KINDS[type(value)].ctype(value)


def cpp_format(template: str, keys: Dict[str, Any]) -> str:
    """Replace every `{KEY}` by its value; other braces are C++ and stay untouched (template.py:61-66)."""
    out = template
    for key, value in keys.items():
        out = out.replace('{' + key + '}', str(value))
    return out


def _param(name: str, arg_type: Any) -> str:
    kind = _KINDS[arg_type]
    return f'{kind.abi_type} {_RAW if kind.abi_type != kind.typed else ""}{name}'


def generate(includes: Iterable[str], arg_defs: Iterable[Tuple], body: str) -> str:
    """Emit the translation unit for one kernel (reference: template.py:69-154).

    `includes` holds `<system>` and `"package"` header names; `arg_defs` is a sequence of `(name, type)`
    with types drawn from the table above; `body` is C++ that sees every argument under its own name
    with its typed C type plus `int& __return_code`.
    """
    assert isinstance(includes, (list, tuple))
    arg_defs = tuple(arg_defs)
    sys_inc = sorted(set(_SYS_INCLUDES) | {i for i in includes if i.startswith('<')})
    pkg_inc = sorted({i for i in includes if i.startswith('"')})

    lines = ['',
             '#define EXPORT_API __attribute__((visibility("default")))',
             '']
    lines += [f'#include {i}' for i in sys_inc] + ['']
    lines += [f'#include {i}' for i in pkg_inc] + ['']
    params = [_param(n, t) for n, t in arg_defs] + ['int& __return_code']
    lines.append(f'extern "C" EXPORT_API void launch({", ".join(params)}) {{')
    lines.append('    // Cast raw types (if needed)')
    for name, arg_type in arg_defs:
        kind = _KINDS[arg_type]
        if kind.abi_type != kind.typed:
            lines.append(f'    auto {name} = reinterpret_cast<{kind.typed}>({_RAW}{name});')
    code = '\n'.join(lines) + '\n'
    code += '\n'.join(('    ' + ln if ln else ln) for ln in body.split('\n'))
    code += '}\n\n'

    if os.getenv('YAN_JIT_DEBUG'):
        print(f'Generated code:\n{code}')
    return code
