from wtconv_amd.modules import WTConv2d, _ScaleModule  # noqa: F401
