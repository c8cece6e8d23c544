from tokasaurus_amd.models.registry import (  # noqa: F401
    ARCHITECTURES,
    Architecture,
    architecture_of,
    build_model,
    config_from_folder,
    register_architecture,
)
from tokasaurus_amd.models.spec import ModelSpec, RunEntry  # noqa: F401
