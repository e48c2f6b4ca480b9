"""Vendor declaration(s) to drop into coffin's ``backends/vendors/`` directory."""
