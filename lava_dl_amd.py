"""Import shim: makes the directory ``lava-dl_amd/`` (not a valid python
identifier) importable as the package ``lava_dl_amd``, so that

    import lava_dl_amd.slayer as slayer

gives the same attribute paths as ``import lava.lib.dl.slayer as slayer`` for
the operators this repository implements."""
import os as _os

__path__ = [_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), 'lava-dl_amd')]
