"""Type-name placeholders: `typename.DT` stands for "some element type" in a
`Buffer[...]` annotation (python/hckernel/typename.py:12-29).  The same name
always yields the same object."""


class Typename:
    def __init__(self, name: str):
        self.name = name

    def __repr__(self) -> str:
        return f"typename.{self.name}"


class _TypenameNamespace:
    def __init__(self):
        self._known = {}

    def __getattr__(self, name: str) -> Typename:
        if name.startswith("__"):
            raise AttributeError(name)
        return self._known.setdefault(name, Typename(name))


typename = _TypenameNamespace()
