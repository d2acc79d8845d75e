"""Import alias so that the reference's `from xmc_classifiers.<module> import <Class>` lines
(src/model.py:146-154) resolve to the MI355X implementation."""
