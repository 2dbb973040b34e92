from . import Max, Sum  # noqa: F401
