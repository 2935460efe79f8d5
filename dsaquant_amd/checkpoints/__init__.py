from . import packed_checkpoint  # noqa: F401
