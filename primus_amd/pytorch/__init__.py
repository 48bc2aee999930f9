"""Operator surface of the MX linear path, laid out like the package the
reference imports (``primus_turbo.pytorch``: ``core``, ``ops``, ``kernels``)."""

from . import core, kernels, ops  # noqa: F401
