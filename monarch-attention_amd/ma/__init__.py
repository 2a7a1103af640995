"""MonarchAttention forward pass for AMD MI355X (gfx950).

Same import surface as the reference's ``ma`` package: put the directory that
contains this package on ``sys.path`` and use

    from ma.monarch_attention import MonarchAttention, PadType, register_impl
"""
