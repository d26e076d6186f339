"""``python -m trifast.tune`` / the ``trifast-tune`` entry point (reference pyproject.toml:36-37)."""

from trifast_amd.tune import *  # noqa: F401,F403
from trifast_amd.tune import main

if __name__ == "__main__":
    main()
