"""Import shim: exposes the package directory ``dflash-mlx_amd/`` (whose name is
not a valid Python identifier) as the importable package ``dflash_mlx_amd``.

``import dflash_mlx_amd`` then behaves like a normal package import; submodules
(``dflash_mlx_amd.verify_qmm`` ...) resolve inside ``dflash-mlx_amd/``.
"""
import os as _os

_PKG_DIR = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "dflash-mlx_amd")
__path__ = [_PKG_DIR]
with open(_os.path.join(_PKG_DIR, "__init__.py"), "r", encoding="utf-8") as _f:
    exec(compile(_f.read(), _os.path.join(_PKG_DIR, "__init__.py"), "exec"), globals())
del _f, _os
