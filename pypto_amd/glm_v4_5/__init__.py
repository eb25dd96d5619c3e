"""Operators named after the reference's models/glm_v4_5 samples."""
