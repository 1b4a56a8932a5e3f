"""trak_amd: the JL gradient-projection and scoring hot path of TRAK on AMD MI355X.

Exposes the reference's plug-in classes (trak/projectors.py, trak/score_computers.py) and
its `fast_jl` function namespace on top of libtrakhip.so (HIP kernels for gfx950).
"""
from . import fast_jl
from .projectors import (
    AbstractProjector,
    ChunkedCudaProjector,
    CudaProjector,
    NoOpProjector,
    ProjectionType,
)
from .featurize import FeatureWriter
from .savers import AbstractSaver, MmapSaver, ModelIDException
from .score_computers import AbstractScoreComputer, BasicScoreComputer, ScoreAccumulator
from .utils import get_matrix_mult, get_parameter_chunk_sizes, vectorize

__all__ = [
    "fast_jl",
    "AbstractProjector",
    "ChunkedCudaProjector",
    "CudaProjector",
    "NoOpProjector",
    "ProjectionType",
    "AbstractScoreComputer",
    "BasicScoreComputer",
    "ScoreAccumulator",
    "FeatureWriter",
    "AbstractSaver",
    "MmapSaver",
    "ModelIDException",
    "get_matrix_mult",
    "get_parameter_chunk_sizes",
    "vectorize",
]
