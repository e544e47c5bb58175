"""Error kinds of the engine.

The reference reports failures as a status code plus a message that names the
key or tensor at fault (`include/liyab/types.h` ErrorCode; messages built in
`src/compat/architecture.cpp:578-596` and `src/core/transformer.cpp:1052-1072`).
Here each code is an exception class, so callers can catch by kind.
"""


class LiyabError(Exception):
    """Base of every error the engine raises on purpose."""


class InvalidModel(LiyabError):
    """config.json or the weights file is malformed or inconsistent."""


class Unsupported(LiyabError):
    """A well-formed request for something this engine does not do."""


class InvalidArgument(LiyabError):
    """A caller's argument is out of range (token id, empty prompt, ...)."""


class ContextFull(LiyabError):
    """A request would pass the model's positions or the configured context."""


class OutOfPages(LiyabError):
    """The page pool cannot hold what a step needs; nothing was committed."""


class Busy(LiyabError):
    """No request slot or state slot is free."""


class KernelError(LiyabError):
    """A HIP launcher refused its operands or the runtime reported an error."""
