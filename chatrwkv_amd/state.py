"""State list shared by the model classes."""


class StateList(list):
    """The state list returned by forward(): a plain list of tensors (model.py:1448-1471) that
    also remembers the flat buffers its entries are views of, so that a one-token step on the
    same state can replay a captured HIP graph."""
    flat = None      # tuple of backing tensors
    views = None     # the tensors as handed out, to detect replaced entries

    def intact(self):
        v = self.views
        return v is not None and len(v) == len(self) and all(a is b for a, b in zip(self, v))
