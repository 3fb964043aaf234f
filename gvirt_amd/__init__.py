"""gvirt_amd — MI355X (gfx950) implementation of Xlite's attention operators.

`gvirt_amd._C` mirrors the attention part of the reference's `xlite._C` extension;
`install_as_xlite()` registers it under that name so reference-style scripts
(`from xlite._C import Runtime, attention`) run unchanged.
"""
import sys
import types


def install_as_xlite() -> None:
    from . import _C
    pkg = sys.modules.get("xlite") or types.ModuleType("xlite")
    pkg._C = _C
    sys.modules["xlite"] = pkg
    sys.modules["xlite._C"] = _C
