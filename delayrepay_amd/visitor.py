"""Name-dispatch visitor over expression nodes (cf. delayrepay/visitor.py:4-24).

`visit(node)` calls `visit_<ClassName>`; a list is visited element by
element; a node without a handler is handed to `default_visit`, which
returns it unchanged.  Handlers are looked up once per class and cached.
"""


class Visitor:
    def __init__(self):
        self._handlers = {}

    def visit(self, node):
        if isinstance(node, list):
            return [self.visit(child) for child in node]
        cls = node.__class__
        try:
            handler = self._handlers[cls]
        except (KeyError, AttributeError):
            if not hasattr(self, "_handlers"):
                self._handlers = {}
            handler = getattr(self, "visit_" + cls.__name__, self.default_visit)
            self._handlers[cls] = handler
        return handler(node)

    def default_visit(self, node):
        return node
