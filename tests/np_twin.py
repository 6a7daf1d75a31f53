"""Independent numpy-float32 re-derivation of the two scale searches.

Written from the published description of the algorithms (the Candle/ggml
``make_qkx1_quants`` / ``make_qx_quants`` family with round-half-away-from-zero),
in explicit scalar loops over ``np.float32`` values so that every operation is one
IEEE binary32 operation.  It shares no code with the C oracle; agreement of the two
on random inputs guards against C-specific slips (implicit double promotion,
contraction, integer overflow, wrong clamp order).
"""
import numpy as np

F = np.float32


def rnd(v):
    """round half away from zero, saturating to i32, NaN -> 0"""
    v = F(v)
    if np.isnan(v):
        return 0
    t = np.trunc(v)
    if abs(F(v - t)) >= F(0.5):
        t = t + np.copysign(F(1.0), v)
    return int(max(min(t, 2147483647), -2147483648))


def qkx1(nmax, ntry, x):
    x = [F(v) for v in x]
    n = len(x)
    L = [0] * n
    lo, hi = min(x), max(x)
    if hi == lo:
        return F(0), F(0)
    lo = min(lo, F(0))
    iscale = F(F(nmax) / F(hi - lo))
    scale = F(F(1) / iscale)
    for _ in range(ntry):
        sumlx, suml2, changed = F(0), 0, False
        for i in range(n):
            li = min(max(rnd(F(iscale * F(x[i] - lo))), 0), nmax)
            if li != L[i]:
                L[i], changed = li, True
            sumlx = F(sumlx + F(F(x[i] - lo) * F(li)))
            suml2 += li * li
        if suml2 == 0:
            break
        scale = F(sumlx / F(suml2))
        s = F(-0.0)
        for i in range(n):
            s = F(s + F(x[i] - F(scale * F(L[i]))))
        lo = F(s / F(n))
        if lo > 0:
            lo = F(0)
        iscale = F(F(1) / scale)
        if not changed:
            break
    return scale, F(-lo)


def qx(n, nmax, x, rmse_type):
    x = [F(v) for v in x[:n]]
    ls = [0] * n
    mx, amax = F(0), F(0)
    for v in x:
        if abs(v) > amax:
            amax, mx = abs(v), v
    if amax == 0:
        return F(0), ls
    iscale = F(F(-nmax) / mx)
    cl = lambda l: min(max(l, -nmax), nmax - 1)
    if rmse_type == 0:
        return F(F(1) / iscale), [nmax + cl(rnd(F(iscale * v))) for v in x]
    wt = rmse_type % 2
    W = [F(v * v) if wt == 1 else F(1) for v in x]
    sumlx, suml2 = F(0), F(0)
    for i in range(n):
        l = cl(rnd(F(iscale * x[i])))
        ls[i] = l + nmax
        sumlx = F(sumlx + F(F(W[i] * x[i]) * F(l)))
        suml2 = F(suml2 + F(W[i] * F(l * l)))
    scale = F(sumlx / suml2)
    best = F(scale * sumlx)
    for _ in range(3):
        isc = F(F(1) / scale)
        slx, sl2, changed = F(0), F(0), False
        for i in range(n):
            l = cl(rnd(F(isc * x[i])))
            if l + nmax != ls[i]:
                changed = True
            slx = F(slx + F(F(W[i] * x[i]) * F(l)))
            sl2 = F(sl2 + F(W[i] * F(l * l)))
        if (not changed) or sl2 == 0 or F(slx * slx) <= F(best * sl2):
            break
        for i in range(n):
            ls[i] = nmax + cl(rnd(F(isc * x[i])))
        sumlx, suml2 = slx, sl2
        scale = F(sumlx / suml2)
        best = F(scale * sumlx)
    for _ in range(5):
        nch = 0
        for i in range(n):
            l = ls[i] - nmax
            slx = F(sumlx - F(F(W[i] * x[i]) * F(l)))
            if slx > 0:
                sl2 = F(suml2 - F(W[i] * F(l * l)))
                nl = cl(rnd(F(F(x[i] * sl2) / slx)))
                if nl != l:
                    slx = F(slx + F(F(W[i] * x[i]) * F(nl)))
                    sl2 = F(sl2 + F(W[i] * F(nl * nl)))
                    if sl2 > 0 and F(F(slx * slx) * suml2) > F(F(sumlx * sumlx) * sl2):
                        ls[i] = nmax + nl
                        sumlx, suml2 = slx, sl2
                        scale = F(sumlx / suml2)
                        nch += 1
        if nch == 0:
            break
    return scale, ls
