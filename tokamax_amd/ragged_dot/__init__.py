"""Ragged dot: operator API (`api`), op base (`base`) and the gfx950 backend (`hip`)."""
