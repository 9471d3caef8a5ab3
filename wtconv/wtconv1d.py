from wtconv_amd.modules import WTConv1d, _ScaleModule  # noqa: F401
