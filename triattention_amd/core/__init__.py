"""Dense (non-paged) scoring and compression API: the reference's core/ package surface."""
