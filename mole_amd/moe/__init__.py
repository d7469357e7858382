from .layer import MOLEModule  # noqa: F401
