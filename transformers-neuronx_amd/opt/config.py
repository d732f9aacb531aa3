"""OPT's configuration (kept under the reference's module path, opt/config.py)."""
from ..config.model_config import OPTConfig  # noqa: F401
