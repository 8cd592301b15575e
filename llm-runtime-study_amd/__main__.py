"""`python -m llm_runtime_study_amd` runs the command line."""

import sys

from .cli import main

if __name__ == "__main__":
    sys.exit(main())
