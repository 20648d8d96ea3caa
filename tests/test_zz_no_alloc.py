"""The allocation-free soft-capped argmax (`ksh_softcap_argmax_static`) against the entry point it is a variant of
(`ksh_kernel_get(KSH_SOFTCAP_ARGMAX)` + `ksh_encode`), through the C ABI: two calls in a row on one context, the
second with a smaller input, so that what the first call left in the shared partial-result array must not leak
into the second; index-exact, as for every integer result."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip

pytestmark = pytest.mark.gpu


def test_static_argmax_equals_the_allocating_entry_point_twice_in_a_row():
    ctx, eng = hip.Context(), hip.Eng()
    try:
        rng = np.random.default_rng(77)
        # first call: the LM head's size, the winner in the last workgroup's share, every partial slot in use
        n1 = 262144
        x1 = (rng.standard_normal(n1) * 8).astype(np.float32)
        x1[n1 - 5] = 90.0
        x1[n1 - 3] = 90.0                                 # a tie: the lower index wins
        # second call: smaller (fewer partial slots written), winner early, all values far below the first call's
        n2 = 1000
        x2 = (rng.standard_normal(n2) - 50.0).astype(np.float32)
        x2[17] = -20.0
        for cap in (30.0, 0.0):
            results = []
            for n, x in ((n1, x1), (n2, x2)):
                bx, b_ref, b_new = ctx.buffer_f32(x), ctx.buffer_f32(np.full(1, -1.0, np.float32)), ctx.buffer_f32(np.full(3, -1.0, np.float32))
                eng.softcap_argmax(ctx, n, cap, bx, b_ref)
                eng.softcap_argmax_static(ctx, n, cap, bx, b_new, out_off=8)
                ctx.synchronize()
                ref, new = ctx.read_f32(b_ref, 1), ctx.read_f32(b_new, 3)
                assert new[0] == -1.0 and new[1] == -1.0          # only the addressed float is written
                assert int(new[2]) == int(ref[0]) == oracle.softcap_argmax(x, cap), (n, cap, new, ref)
                results.append(int(new[2]))
                for b in (bx, b_ref, b_new):
                    b.release()
            assert results == [n1 - 5, 17]
        # an offset into the input: the slice [off, off + n)
        bx, bo = ctx.buffer_f32(x1), ctx.buffer_empty_f32(1)
        eng.softcap_argmax_static(ctx, 5000, 30.0, bx, bo, x_off=4 * 1000)
        ctx.synchronize()
        assert int(ctx.read_f32(bo, 1)[0]) == oracle.softcap_argmax(x1[1000:6000], 30.0)
        # sizes beyond the stated maximum and bindings that do not fit are refused
        with pytest.raises(hip.KshError, match="outside"):
            eng.softcap_argmax_static(ctx, 1 << 24, 30.0, bx, bo)
        with pytest.raises(hip.KshError, match="outside"):
            eng.softcap_argmax_static(ctx, 0, 30.0, bx, bo)
        with pytest.raises(hip.KshError, match="x needs"):
            eng.softcap_argmax_static(ctx, n1, 30.0, bx, bo, x_off=4)
        with pytest.raises(hip.KshError, match="out needs"):
            eng.softcap_argmax_static(ctx, n1, 30.0, bx, bo, out_off=4)
    finally:
        ctx.close()
