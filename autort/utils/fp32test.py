"""``python -m autort.utils.fp32test``: see antares_amd.autort.utils.fp32test."""
import sys

from antares_amd.autort.utils.fp32test import *          # noqa: F401,F403
from antares_amd.autort.utils.fp32test import main

if __name__ == '__main__':
    sys.exit(main())
