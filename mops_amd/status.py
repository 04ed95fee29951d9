"""Error type raised when a C-ABI call reports a failure.

Same contract as ``python/mops/src/mops/status.py:25-38`` of lab-cosmo/mops:
a non-zero status becomes an exception carrying the library's last error
message and the status code.
"""


class MopsError(Exception):
    """A ``mops_*`` entry point returned a non-zero status."""

    def __init__(self, message, status=None):
        super().__init__(message)
        self.message = message
        self.status = status
