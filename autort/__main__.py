"""``python -m autort --ir ... -i ... -c ...`` (README.md:75-77)."""
import sys

from antares_amd.autort.cli import main

sys.exit(main())
