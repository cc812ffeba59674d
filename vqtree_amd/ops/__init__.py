"""Operator modules mirroring the reference's `ops/` package, backed by libvqattn_gfx950."""
