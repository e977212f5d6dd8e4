"""Layers are put together from parts; see ``clockwork_amd.parts.base`` for the interfaces."""
