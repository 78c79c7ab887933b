"""User-written masks: build and load a library around one mask functor.

The reference lets a user subclass ``ChillMask`` with Triton static methods and compiles them on
first use ("Creating Your Own Mask", README.md:124-179; registration chill.py:27-58).  Here the
device statement of a user mask is a small C++ functor (the contract is documented in
``csrc/chill_user_mask.h``), compiled by ``hipcc`` together with the same kernel templates the
built-in masks use into a library of its own that serves mask id ``MASK_USER``:

    class SinkWindowChillMask(ChillMask):
        hip_functor = '''
            static constexpr int kNumArgs = 2;
            static constexpr bool kMonotoneLimits = false;
            CHILL_HD static bool pred(int q, int k, int, MaskArgs a) { ... }
            CHILL_HD static Range k_range_for_q(int q, int seq_len, MaskArgs a) { ... }
            CHILL_HD static Range q_range_for_k(int k, int seq_len, MaskArgs a) { ... }
        '''
        def __init__(self, sinks, window): super().__init__((sinks, window))
        # numpy statements of the same rules, for verify():
        @staticmethod
        def mask(q, k, seq_len, args): ...

``hip_functor`` is the BODY of ``chill::Mask<CHILL_MASK_USER>``; alternatively ``hip_header`` names a
complete header file.  The library is built once per (class name, functor text, kernel sources) under
``chill-attention_amd/lib/user/`` and loaded from there afterwards; building needs ``hipcc`` and
``make`` and takes about 15 s.  ``ChillMask.verify`` checks the numpy rules against the compiled
functor, so a wrong functor does not go unnoticed.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import typing

from . import _lib

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG_DIR)
CSRC_DIR = os.path.join(_ROOT, "csrc")
USER_LIB_DIR = os.path.join(_ROOT, "lib", "user")
USER_BUILD_DIR = os.path.join(_ROOT, "build", "user")

_WRAPPER = """// generated from {cls}.hip_functor
#pragma once
namespace chill {{
template <>
struct Mask<CHILL_MASK_USER> : MaskDefaults {{
{body}
}};
}}  // namespace chill
"""

_loaded: dict = {}


def is_user_mask(cls) -> bool:
    return cls.mask_id is None and (getattr(cls, "hip_functor", None) or getattr(cls, "hip_header", None)) is not None


def functor_source(cls) -> str:
    """Text of the header that specialises ``chill::Mask<CHILL_MASK_USER>`` for ``cls``."""
    header = getattr(cls, "hip_header", None)
    if header:
        with open(header) as f:
            return f.read()
    return _WRAPPER.format(cls=cls.__name__, body=cls.hip_functor)


def _kernel_sources_digest() -> bytes:
    h = hashlib.sha1()
    for name in sorted(os.listdir(CSRC_DIR)):
        # (the generated .inc files follow from the .py generators)
        if name.endswith((".h", ".hip", ".cpp", ".py")) or name == "Makefile":
            with open(os.path.join(CSRC_DIR, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.digest()


def _key(cls) -> str:
    """One library per (class, functor text, kernel sources): editing either builds a new one."""
    digest = hashlib.sha1(functor_source(cls).encode() + _kernel_sources_digest()).hexdigest()[:12]
    return f"{cls.__name__}-{digest}"


def library_path(cls) -> str:
    return os.path.join(USER_LIB_DIR, _key(cls), "libchill_attention_hip.so")


def build(cls, force: bool = False, jobs: int = 8) -> str:
    """Compile the library of user mask ``cls`` (if it is not there yet) and return its path."""
    path = library_path(cls)
    if os.path.exists(path) and not force:
        return path
    if shutil.which("hipcc") is None or shutil.which("make") is None:
        raise RuntimeError(
            f"{cls.__name__}: its library {path} has not been built and hipcc / make are not on PATH"
        )
    build_dir = os.path.join(USER_BUILD_DIR, _key(cls))
    os.makedirs(build_dir, exist_ok=True)
    header = os.path.join(build_dir, "user_mask.h")
    with open(header, "w") as f:
        f.write(functor_source(cls))
    cmd = ["make", "-C", CSRC_DIR, f"-j{jobs}", f"USER_MASK={header}", f"BUILD={build_dir}",
           f"LIBDIR={os.path.dirname(path)}"]
    if force:
        cmd.insert(1, "-B")
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0 or not os.path.exists(path):
        raise RuntimeError(f"{cls.__name__}: building the mask library failed:\n{res.stdout[-4000:]}")
    # the 16-bit head-dim-256 kernels name accumulation registers themselves: make sure the compiler kept
    # out of them with this functor inlined
    from . import tune

    try:
        tune.check_hand_managed_registers({"CHILL_USER_MASK_HEADER": f'"{header}"'})
    except RuntimeError as e:
        os.remove(path)
        raise RuntimeError(f"{cls.__name__}: simplify the functor: {e}") from e
    # libraries of this class built from older sources (another key) are of no use any more
    for root in (USER_BUILD_DIR, os.path.dirname(os.path.dirname(path))):
        for name in os.listdir(root):
            if name.startswith(cls.__name__ + "-") and name != _key(cls):
                shutil.rmtree(os.path.join(root, name), ignore_errors=True)
    return path


def library_for(cls) -> typing.Any:
    """The loaded library of user mask ``cls`` (built first if necessary)."""
    key = _key(cls)
    if key not in _loaded:
        lib = _lib.load_library(build(cls))
        if lib.chill_has_user_mask() != 1:
            raise RuntimeError(f"{library_path(cls)} was not built around a user mask")
        _loaded[key] = lib
    return _loaded[key]
