"""The three kernel modules of the reference's ``cornstarch/kernel`` package, served by ``cornstarch_amd.kernel``."""
