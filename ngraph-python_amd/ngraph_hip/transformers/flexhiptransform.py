"""`flexhip`: flex16 variant of the HIP transformer (filled in below)."""
