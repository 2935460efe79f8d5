from . import vdm_w4a4  # noqa: F401
