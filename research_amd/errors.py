"""Exception types of the host layer (names follow jaxtitan/errors.py)."""


class JtmoeError(Exception):
    """Base class."""


class ContractError(JtmoeError):
    """Raised when an argument or an artefact violates the layer's contract."""


class KernelLaunchError(JtmoeError):
    """Raised when the native library reports a launch failure."""
