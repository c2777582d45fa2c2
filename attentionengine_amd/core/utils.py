"""Small helpers shared by the frontend.

``meta_tensor`` mirrors attention_engine/core/utils.py:44-51: a shape-and-dtype record in
(B, H, S, D) order used to describe q/k/v at construction time (runtime tensors are
[B, S, H, D]).
"""


class meta_tensor:
    """Shape/dtype descriptor: ``meta_tensor(B, H, S, D, dtype=torch.float16)``.
    Dimensions may be strings for dynamic extents (attn_script/mha.py:90-95)."""

    def __init__(self, *shape, **kwargs):
        self.shape = shape
        self.kargs = kwargs

    @property
    def dtype(self):
        return self.kargs["dtype"]

    def __repr__(self):
        return f"meta_tensor{self.shape}[{self.kargs.get('dtype')}]"


class IndentedCode:
    """Line buffer with an indentation level (same role as core/utils.py:4-36)."""

    def __init__(self, indent: int = 0):
        self.indent = indent
        self.code = ""

    def __str__(self):
        return self.code

    def add_line(self, line: str):
        self.code += "    " * self.indent + line + "\n"

    def __iadd__(self, other):
        if isinstance(other, str):
            self.add_line(other)
        else:
            for line in str(other).split("\n"):
                if line:
                    self.add_line(line)
        return self

    def more_indent(self, n: int = 1):
        self.indent += n

    def less_indent(self, n: int = 1):
        self.indent -= n
