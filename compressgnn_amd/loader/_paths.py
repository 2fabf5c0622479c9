"""Puts the package directories that hold the bare-name modules (compressgnn_runtime,
compressgnn_offline, the layer and loader modules) on sys.path, the way the reference's
scripts extend sys.path with its layer/ and loader/ directories."""
import os
import sys

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for _p in (PKG, os.path.join(PKG, "loader"), os.path.join(PKG, "layer")):
    if _p not in sys.path:
        sys.path.append(_p)
