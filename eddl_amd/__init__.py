"""eddl_amd - MI355X (gfx950) backend for the CNN forward path of EDDL.

``libeddlhip.so`` (HIP kernels behind a C ABI, see include/eddlhip.h) is the product; this
package is the Python host side used by the tests and the benchmark: a ctypes binding
(:class:`Backend`, :class:`DeviceTensor`), mirrors of the reference's descriptors
(:mod:`eddl_amd.descriptors`) and forward-only model graphs (:mod:`eddl_amd.net`,
:mod:`eddl_amd.models`).
"""
from .backend import Backend, DeviceTensor, EddlHipError  # noqa: F401
