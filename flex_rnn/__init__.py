"""Drop-in alias: `import flex_rnn` resolves to the MI355X backend with the reference's
public names (/root/reference/flex_rnn/__init__.py:1-3)."""
from flex_rnn_amd import jit, check_grad, benchmark, __version__  # noqa: F401
