"""Drop-in name: `import arboretum` resolves to the MI355X implementation."""
from arboretum_amd import *  # noqa: F401,F403
from arboretum_amd import __all__  # noqa: F401
