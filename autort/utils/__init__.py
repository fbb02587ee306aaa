"""Drop-in import name for the device check-up programs: ``python -m autort.utils.memtest`` and friends."""
from antares_amd.autort.utils import *          # noqa: F401,F403
