from . import primary  # noqa: F401
