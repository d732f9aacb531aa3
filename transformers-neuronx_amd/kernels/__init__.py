"""Kernel backends: `hip` is the product path, `reference` its plain torch rendition."""


def make_ops(kind: str, dtype, device):
    if kind == "reference":
        from .reference import ReferenceOps
        return ReferenceOps(dtype, device)
    if kind == "hip":
        from .hip import HipOps
        return HipOps(dtype, device)
    raise ValueError(f"unknown kernel backend {kind!r}")
