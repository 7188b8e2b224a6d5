"""Stand-ins for the reference's native modules, for code that keeps the reference's own Python layer."""
