"""Host-side runtime: ctypes binding of the C-ABI library, module cache."""
