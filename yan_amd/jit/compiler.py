"""hipcc backend of the JIT: compiler discovery, source hashing, on-disk kernel cache, atomic install.

Keeps the behaviour of the reference's `yan/jit/compiler.py` (`get_nvcc_compiler` :56-96, cache dirs :100-128,
`put` :131-151, `build` :154-253) with the backend re-targeted to gfx950:

* a kernel lives in `<cache>/cache/kernel.<name>.<md5[:12]>/{kernel.cu,kernel.args,kernel.so}`;
* the key hashes name, package-header digest, generated code, compiler (path, version) and flags;
* files are written to `<cache>/tmp` first and renamed into place, so concurrent processes may race on the
  same kernel and each still ends up with a complete directory;
* a failed compile raises `RuntimeError`.

The code object is always built for gfx950 (`YAN_OFFLOAD_ARCH` overrides), which is what lets a kernel be
built on a machine without a GPU and loaded on one with it.
"""
import functools
import hashlib
import os
import re
import shutil
import subprocess
import uuid
from typing import List, Tuple

from .runtime import Runtime, RuntimeCache
from .template import typename_map

runtime_cache = RuntimeCache()

_HEADER_SUFFIXES = ('.h', '.hpp', '.cuh')
_MIN_HIP_VERSION = (6, 4)


def hash_to_hex(s: str) -> str:
    return hashlib.md5(s.encode('utf-8')).hexdigest()[:12]


@functools.lru_cache(maxsize=None)
def get_jit_include_dir() -> str:
    return os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', 'include'))


@functools.lru_cache(maxsize=None)
def get_yan_version() -> str:
    """Digest of every kernel header shipped with the package; editing a header invalidates the cache."""
    root = get_jit_include_dir()
    assert os.path.isdir(root), f'Cannot find the kernel include directory {root}'
    paths: List[str] = []
    for base, _, files in os.walk(root):
        paths += [os.path.join(base, f) for f in files if f.endswith(_HEADER_SUFFIXES)]
    md5 = hashlib.md5()
    for p in sorted(paths):
        md5.update(os.path.relpath(p, root).encode())
        with open(p, 'rb') as f:
            md5.update(f.read())
    return md5.hexdigest()[:12]


@functools.lru_cache(maxsize=None)
def get_hipcc_compiler() -> Tuple[str, str]:
    """Locate hipcc and return `(path, 'major.minor')`; `YAN_HIPCC_COMPILER` (or the reference's
    `YAN_NVCC_COMPILER`) names a specific binary."""
    candidates = [os.getenv('YAN_HIPCC_COMPILER'), os.getenv('YAN_NVCC_COMPILER')]
    rocm = os.getenv('ROCM_PATH') or os.getenv('ROCM_HOME') or '/opt/rocm'
    candidates += [os.path.join(rocm, 'bin', 'hipcc'), shutil.which('hipcc')]
    pattern = re.compile(r'HIP version:\s*(\d+)\.(\d+)')
    for path in candidates:
        if not path or not os.path.exists(path):
            continue
        try:
            text = subprocess.check_output([path, '--version'], stderr=subprocess.STDOUT, universal_newlines=True)
        except (subprocess.SubprocessError, OSError) as e:
            print(f'Error checking hipcc version for {path}: {e}')
            continue
        found = pattern.search(text)
        if not found:
            print(f'Cannot determine version for hipcc compiler {path}')
            continue
        version = (int(found.group(1)), int(found.group(2)))
        if version >= _MIN_HIP_VERSION:
            return path, f'{version[0]}.{version[1]}'
        print(f'hipcc {path} version {version} is lower than {_MIN_HIP_VERSION}')
    raise RuntimeError('Cannot find a hipcc with HIP >= %d.%d; set ROCM_PATH or YAN_HIPCC_COMPILER' % _MIN_HIP_VERSION)


# Callers written against the reference ask for the compiler under this name.
get_nvcc_compiler = get_hipcc_compiler


def get_offload_arch() -> str:
    return os.getenv('YAN_OFFLOAD_ARCH', 'gfx950')


def get_default_user_dir() -> str:
    path = os.getenv('YAN_CACHE_DIR')
    if path:
        os.makedirs(path, exist_ok=True)
        return path
    return os.path.expanduser('~/.cache/yan')


def get_tmp_dir() -> str:
    return os.path.join(get_default_user_dir(), 'tmp')


def get_cache_dir() -> str:
    return os.path.join(get_default_user_dir(), 'cache')


def make_tmp_dir() -> str:
    tmp = get_tmp_dir()
    os.makedirs(tmp, exist_ok=True)
    return tmp


def _install(tmp_path: str, path: str) -> None:
    try:
        os.replace(tmp_path, path)
    except OSError:          # e.g. tmp and cache on different file systems
        shutil.copy2(tmp_path, path)
        os.unlink(tmp_path)


def put(path: str, data, is_binary: bool = False) -> None:
    """Write `data` to `path` so that readers see either the old file or the complete new one."""
    tmp_path = os.path.join(make_tmp_dir(), f'file.tmp.{uuid.uuid4()}.{hash_to_hex(path)}')
    with open(tmp_path, 'wb' if is_binary else 'w') as f:
        f.write(data)
    _install(tmp_path, path)


def get_compile_flags() -> List[str]:
    flags = ['-std=c++20', '-O3', f'--offload-arch={get_offload_arch()}', '-shared', '-fPIC',
             '-fno-gpu-rdc', '-Wno-unused-command-line-argument', '-Wno-deprecated-declarations',
             # keep fp32 arithmetic on the scalar-per-lane VALU forms
             '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']
    if os.getenv('YAN_SAVE_TEMPS'):
        flags.append('-save-temps')
    return flags


def kernel_dir(name: str, code: str) -> str:
    """Cache directory a (name, code) pair maps to under the current compiler, flags and headers."""
    signature = f'{name}$${get_yan_version()}$${code}$${get_hipcc_compiler()}$${get_compile_flags()}'
    return os.path.join(get_cache_dir(), f'kernel.{name}.{hash_to_hex(signature)}')


def build(name: str, arg_defs: tuple, code: str) -> Runtime:
    path = kernel_dir(name, code)
    cached = runtime_cache[path]
    if cached is not None:
        if os.getenv('YAN_JIT_DEBUG'):
            print(f'Using cached JIT runtime {os.path.basename(path)} during build')
        return cached

    os.makedirs(path, exist_ok=True)
    src_path = os.path.join(path, 'kernel.cu')
    put(os.path.join(path, 'kernel.args'), ', '.join(f"('{n}', {typename_map[t]})" for n, t in arg_defs))
    put(src_path, code)

    lib_path = os.path.join(path, 'kernel.so')
    tmp_lib_path = os.path.join(make_tmp_dir(), f'hipcc.tmp.{uuid.uuid4()}.{hash_to_hex(lib_path)}.so')
    # `.cu` is the cache contract's file name; `-x hip` tells hipcc what is inside.
    command = [get_hipcc_compiler()[0], '-x', 'hip', src_path, '-o', tmp_lib_path,
               *get_compile_flags(), f'-I{get_jit_include_dir()}']
    if os.getenv('YAN_JIT_DEBUG') or os.getenv('YANJIT_PRINT_HIPCC_COMMAND') or os.getenv('YANJIT_PRINT_NVCC_COMMAND'):
        print(f'Compiling JIT runtime {os.path.basename(path)} with command {command}')
    try:
        done = subprocess.run(command, cwd=make_tmp_dir(), stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                              universal_newlines=True)
    except OSError as e:
        raise RuntimeError(f'Failed to compile {src_path}: {e}')
    if done.returncode != 0:
        raise RuntimeError(f'Failed to compile {src_path}: hipcc exited with {done.returncode}\n{done.stdout[-4000:]}')
    if os.getenv('YAN_JIT_DEBUG') and done.stdout:
        print(done.stdout)
    _install(tmp_lib_path, lib_path)

    runtime_cache[path] = Runtime(path)
    return runtime_cache[path]
