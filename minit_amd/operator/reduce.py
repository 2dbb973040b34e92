from . import Max, Mean, Sum  # noqa: F401
