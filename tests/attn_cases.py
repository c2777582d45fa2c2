"""The example scripts' user-level definitions live in the package (attn_script); the tests use them
under this name."""
from attn_script import *  # noqa: F401,F403
