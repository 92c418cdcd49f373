"""Host-side counterparts of the reference modules that call the MXFP8 linear path."""
