"""``python -m rapid_llm_amd <command> ...``: the command line of ``rapid_llm_amd.cli``."""

import sys

from .cli import main

sys.exit(main())
