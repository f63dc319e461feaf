"""Backend protocol (BackendBench/backends/base.py:8-10): a name, `op in backend`, `backend[op]`."""


class Backend:
    def __init__(self, name):
        self.name = name
