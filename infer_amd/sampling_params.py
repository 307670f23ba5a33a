"""What a request asks of the sampler and of the stop test.

Same three fields, names and defaults as the reference's ``infer/sampling_params.py:3-8`` (callers pass them
positionally or by keyword); here the values are checked when the object is built, because a negative
temperature or a zero token budget otherwise surfaces steps later as a division or an endless request."""


class SamplingParams:
    __slots__ = ("temperature", "max_tokens", "ignore_eos")

    def __init__(self, temperature: float = 1.0, max_tokens: int = 64, ignore_eos: bool = False):
        temperature = float(temperature)
        max_tokens = int(max_tokens)
        if not temperature >= 0.0:
            raise ValueError(f"temperature must be >= 0, got {temperature}")
        if max_tokens < 1:
            raise ValueError(f"max_tokens must be >= 1, got {max_tokens}")
        self.temperature = temperature
        self.max_tokens = max_tokens
        self.ignore_eos = bool(ignore_eos)

    @property
    def greedy(self) -> bool:
        """Temperature 0 selects the arg-max token."""
        return self.temperature == 0.0

    def _key(self):
        return (self.temperature, self.max_tokens, self.ignore_eos)

    def __eq__(self, other):
        return isinstance(other, SamplingParams) and self._key() == other._key()

    def __hash__(self):
        return hash(self._key())

    def __repr__(self):
        return "SamplingParams(temperature=%r, max_tokens=%r, ignore_eos=%r)" % self._key()
