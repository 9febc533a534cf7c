from .base import ModelConfig, field_from_json  # noqa: F401
from .registry import (  # noqa: F401
    Architecture, register_architecture, architecture_for, registered_architectures,
    load_config,
)
from .llama import LlamaConfig  # noqa: F401
from .mamenex import MamenexConfig  # noqa: F401
from .nagezen import NagezenConfig  # noqa: F401
from .milenex import MilenexConfig  # noqa: F401
from .lagusun import LagusunConfig  # noqa: F401
