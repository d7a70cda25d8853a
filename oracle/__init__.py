"""CPU oracle for the flash-decode hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory.  Only the test-suite,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker -- never as the thing being measured or
shipped.  The product path raises when its HIP library is missing; it never
routes through this code.

``oracle/c/ref_decode.c`` is a second, independent restatement of the decode in plain C (built by
``oracle/c/build.py``); tests/test_c_oracle.py holds the two against each other and the C consumer of the ABI
under tests/c_abi/ checks the library against it with no Python in the loop.
"""
from .ref_decode import (  # noqa: F401
    ref_paged_attn,
    ref_paged_attn_lse,
    fp8_e4m3fn_decode_table,
    dequant_fp8_cache,
    quantize_fp8_cache,
)
from .ref_kv_append import (  # noqa: F401
    ref_set_cos_sin_cache,
    ref_rope,
    ref_rms_norm,
    ref_quantize_fp8,
    brute_force_fp8,
    ref_kv_append,
)
from .split_combine_model import (  # noqa: F401
    split_range,
    model_split_kv,
    model_combine,
    model_gqa_fwd_batch_decode,
    model_sp_decode,
)
