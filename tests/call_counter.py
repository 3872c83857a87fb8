"""A helper of the tests: which entry points of `inferrs_amd.ops` a piece of work went through."""


class CallCounter:
    """Counts the calls of some entry points of `inferrs_amd.ops` while it is active (the module's own functions
    look each other up by name, so the wrappers are seen from inside too)."""

    def __init__(self, *names):
        self.names, self.calls, self._saved = names, {n: 0 for n in names}, {}

    def __enter__(self):
        from inferrs_amd import ops
        for n in self.names:
            inner = self._saved[n] = getattr(ops, n)

            def wrapper(*a, _inner=inner, _n=n, **k):
                self.calls[_n] += 1
                return _inner(*a, **k)
            setattr(ops, n, wrapper)
        return self

    def __exit__(self, *exc):
        from inferrs_amd import ops
        for n, fn in self._saved.items():
            setattr(ops, n, fn)
