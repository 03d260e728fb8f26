"""Operator classes of the gfx950 backend (one class per logical op)."""
