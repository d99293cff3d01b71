"""``python -m spite_amd ...`` is the ``spite`` command line."""
import sys

from .cli import main

sys.exit(main())
