"""MI355X-native sparse-retrieval hot path of Unified Cache Management.

``ops``     torch-tensor front end of the C-ABI library ``libucm_hip.so``
``sparse``  host side: the UcmSparseBase hook surface, the retrieval-worker
            submit/poll/wait/get_result object and the GSA/ESA-shaped plugins
            that drive the kernels

The HIP library is required: importing ``ops`` raises if it has not been built
(``python unified-cache-management_amd/build.py``).  There is no CPU fallback.
"""
__version__ = "0.1.0"
