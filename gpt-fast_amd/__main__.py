import sys

from .engine.cli import cli

sys.exit(cli())
