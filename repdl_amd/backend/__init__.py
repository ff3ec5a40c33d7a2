"""Device backends.  ``hip`` is the only one: the MI355X C-ABI library."""
