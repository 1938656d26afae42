"""MI355X-native FlashSinkhorn: streaming entropic OT on hand-written gfx950 kernels."""
__version__ = "0.1.0"
