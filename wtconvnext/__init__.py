from .wtconvnext import WTConvNeXt, wtconvnext_base, wtconvnext_small, wtconvnext_tiny  # noqa: F401
