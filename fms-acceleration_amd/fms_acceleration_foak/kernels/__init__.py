"""Stand-alone accelerated operators of the fast-kernels plugin (namesake of
fms_acceleration_foak/kernels in the reference)."""
