"""MI355X-native array kernels behind AMDGPU.jl's ROCArray: host-side mirror of the Julia API.

The Julia method families of the reference keep their names and argument meaning here
(``mapreducedim_`` for ``mapreducedim!`` etc.); each call goes through the C ABI of ``librk.so``
(include/rk.h) into hand-written gfx950 kernels.  There is no CPU path: importing this package
without the built library raises.
"""
from ._lib import (RKError, DimensionMismatch, UnsupportedError, lib, LIB_PATH)       # noqa: F401
from .array import ROCArray, Array, similar, zeros, workspace                         # noqa: F401
from .mapreduce import (mapreduce, mapreducedim_, sum, prod, maximum, minimum, count, # noqa: F401,A004
                        findmax, findmin, argmax, argmin, extrema, any, all, findfirst, reduce_eltype, identity, abs2, abs_,
                        add_sum, mul_prod, add, mul, max_, min_)
from .accumulate import accumulate, accumulate_, cumsum, cumprod, accumulate_eltype    # noqa: F401
from . import broadcast                                                               # noqa: F401
from .broadcast import (lazy, materialize, materialize_, fill_, Broadcasted,            # noqa: F401
                        isodd, iseven, isnan, ifelse)
from .views import ROCView, view, transpose, PermutedDimsArray                         # noqa: F401
from .volumerhs import volumerhs_                                                     # noqa: F401
from .indexing import findall, getindex_mask                                                         # noqa: F401
from .reverse import reverse, reverse_                                                # noqa: F401
from .permutedims import permutedims, permutedims_                                    # noqa: F401
from .sorting import sort, sort_, sortperm, sortperm_, isless, not_isless             # noqa: F401

__version__ = "0.1.0"
