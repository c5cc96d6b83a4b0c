"""SciPy-named functions on device arrays (``autograd_amd.scipy.special.logsumexp``)."""
