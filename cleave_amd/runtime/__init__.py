"""What happens to a generated kernel: hiprtc, a check against the reference, a timing; the ctypes binding of the native library."""
