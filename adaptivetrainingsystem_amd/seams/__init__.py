"""Shim modules carrying the import names the reference model looks for."""
