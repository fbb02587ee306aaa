"""``python -m autort.utils.export``: see antares_amd.autort.utils.export."""
import sys

from antares_amd.autort.utils.export import *          # noqa: F401,F403
from antares_amd.autort.utils.export import main

if __name__ == '__main__':
    sys.exit(main())
