from .log4Error import invalidInputError, invalidOperationError  # noqa: F401
