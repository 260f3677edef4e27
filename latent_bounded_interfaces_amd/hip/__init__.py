"""Device-kernel wrappers; the counterpart of the reference's ``cuda`` package."""
