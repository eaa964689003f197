"""Import hook target: ``VERL_USE_EXTERNAL_MODULES=verl_amd.plugin`` installs the HIP scoring path.

verl imports every module named in that variable while ``import verl`` runs
(verl/__init__.py:49-52, verl/utils/import_utils.py:81-88), before any engine
module has bound ``logprobs_from_logits`` by name.
"""

from .hook import install

install()
