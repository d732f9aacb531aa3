from .spec import ARCHITECTURE, opt_spec  # noqa: F401
