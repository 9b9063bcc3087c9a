"""Exception types of the data-loading layer (reference errors.py:1-17)."""


class Error(Exception):
    """Root of the package's own exceptions."""


class InputError(Error):
    """Bad input data: an unreadable image, an unexpected label value, stacks of
    different length.  The text is kept in ``message`` as well as in ``args``."""

    def __init__(self, message):
        super().__init__(message)
        self.message = message
