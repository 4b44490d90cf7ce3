"""JIT layer: `generate` writes the source of one `extern "C" launch(...)`, `build` compiles it with hipcc into a
cached `kernel.so`, `Runtime` loads and calls it. The public names are those of the reference's `yan.jit`
(`yan/jit/__init__.py:1-3`); `get_nvcc_compiler` is kept as an alias of `get_hipcc_compiler` for callers that ask for it.
"""
from . import compiler, runtime, template

build = compiler.build
get_hipcc_compiler = compiler.get_hipcc_compiler
get_nvcc_compiler = compiler.get_nvcc_compiler
cpp_format = template.cpp_format
generate = template.generate
Runtime = runtime.Runtime

__all__ = ['build', 'get_hipcc_compiler', 'get_nvcc_compiler', 'cpp_format', 'generate', 'Runtime', 'compiler', 'runtime', 'template']
