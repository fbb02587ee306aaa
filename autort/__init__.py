"""Drop-in import name: ``import autort`` resolves to the MI355X backend."""
from antares_amd.autort import *          # noqa: F401,F403
from antares_amd.autort import ops, export, device, download, profile, ExportedOp   # noqa: F401
