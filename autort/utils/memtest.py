"""``python -m autort.utils.memtest``: see antares_amd.autort.utils.memtest."""
import sys

from antares_amd.autort.utils.memtest import *          # noqa: F401,F403
from antares_amd.autort.utils.memtest import main

if __name__ == '__main__':
    sys.exit(main())
