"""The names of ``flydsl.expr`` that harness code for this path touches: element-type tags for
``from_c_void_p`` and a ``Stream`` wrapper (python/flydsl/expr/typing.py:1273-1285)."""


class _Tag:
    def __init__(self, name):
        self.name = name

    def __repr__(self):
        return f"fx.{self.name}"


Uint8 = _Tag("Uint8")
Int8 = _Tag("Int8")


class Stream:
    """Wraps a raw stream handle or a ``torch.cuda.Stream``."""

    def __init__(self, value=None):
        self.value = int(getattr(value, "cuda_stream", value or 0))

    @property
    def cuda_stream(self):
        return self.value
