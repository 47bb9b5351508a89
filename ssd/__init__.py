"""Import-path alias: ``ssd.bi.ssd_combined`` and ``ssd.modules`` resolve to the MI355X implementation."""
