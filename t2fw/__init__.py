"""Import-compatible alias of the reference's package layout: ``from
t2fw.functional_lfw import LFWFunction`` (README usage of the reference) resolves to
the MI355X implementation in ``t2fw_amd``."""
