"""Name-dispatch visitor over expression nodes (cf. delayrepay/visitor.py:4-24).

`visit(node)` calls `visit_<ClassName>`; a list is visited element by
element; a node without a handler is handed to `default_visit`, which
returns it unchanged.  Handlers are looked up once per (visitor class, node
class) and cached as plain functions on the visitor's class: a cache of bound
methods on the instance would make every visitor part of a reference cycle,
and what it holds (a tracer holds device arrays) would wait for the cycle
collector instead of being freed with its last user.
"""


class Visitor:
    def __init__(self):
        pass

    def visit(self, node):
        if isinstance(node, list):
            return [self.visit(child) for child in node]
        cls = node.__class__
        own = self.__class__
        try:
            handler = own.__dict__["_handlers"][cls]
        except KeyError:
            table = own.__dict__.get("_handlers")
            if table is None:
                table = {}
                own._handlers = table
            handler = getattr(own, "visit_" + cls.__name__, None) or own.default_visit
            table[cls] = handler
        return handler(self, node)

    def default_visit(self, node):
        return node
