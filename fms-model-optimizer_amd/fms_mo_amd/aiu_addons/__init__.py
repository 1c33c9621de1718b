"""Counterparts of the reference's accelerator add-ons that sit on the W8A8 path."""
