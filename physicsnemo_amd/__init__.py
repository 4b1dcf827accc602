"""MI355X-native PhysicsAttention layer of Transolver and its callers (hand-written HIP kernels behind a C ABI)."""
from .physics_attention import (  # noqa: F401
    PhysicsAttentionBase,
    PhysicsAttentionIrregularMesh,
    PhysicsAttentionStructuredMesh2D,
    PhysicsAttentionStructuredMesh3D,
)
from .context_projector import (BQWarp, ContextProjector, GeometricFeatureProcessor,  # noqa: F401
                                MultiScaleFeatureExtractor, StructuredContextProjector)
from .flare import FLARE, FLAREBlock, FLAREModel, GALE_FA  # noqa: F401
from .gale import GALE, GALEBlock, GALEStructuredMesh2D, GALEStructuredMesh3D  # noqa: F401
from .geotransolver import GeoTransolver, GlobalContextBuilder  # noqa: F401
from .graphs import GraphedForward  # noqa: F401
from .transolver import Mlp, Transolver, TransolverBlock  # noqa: F401

__version__ = "0.1.0"
