"""``python -m autort.utils.mmtest``: see antares_amd.autort.utils.mmtest."""
import sys

from antares_amd.autort.utils.mmtest import *          # noqa: F401,F403
from antares_amd.autort.utils.mmtest import main

if __name__ == '__main__':
    sys.exit(main())
