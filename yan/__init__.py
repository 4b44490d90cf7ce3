"""`import yan` for code written against the reference's package name (`yan/__init__.py:3-5` there): the name is an
alias of `yan_amd`, the module object is the same one."""
import sys

import yan_amd

sys.modules[__name__] = yan_amd
