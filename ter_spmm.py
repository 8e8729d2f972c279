"""Import-name shim: ``import ter_spmm`` resolves to ternaryllm_amd.ter_spmm, the module that
replaces the reference's CUDA extension of that name (its four callables, plus `prepare`)."""
from ternaryllm_amd.ter_spmm import (convert_to_ter_csc, convert_to_ter_tiled_csc,  # noqa: F401
                                     convert_to_ter_tiled_mcsc, prepare, ter_spmm)
