"""docc_amd: an MI355X-native `rocm` target for docc's math library nodes.

    from docc_amd.python import native            # @native(target="rocm")
    import docc_amd.torch                          # torch.compile(model, backend="docc")
    from docc_amd import runtime                   # the C-ABI runtime and kernel launchers
"""
__version__ = "0.1"
