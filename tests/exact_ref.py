"""Rational-arithmetic restatement of the reference's scale searches and k-quant block quantizers.

Purpose: expected results for the oracle (and, through the fixtures, for the HIP kernels) that do not come
from running floating-point code.  Every binary32 value is a ``fractions.Fraction`` (plus a sign for zero and
an infinity / NaN tag); every operation computes the exact rational result and rounds it once to binary32 by
the IEEE-754 definition (round to nearest, ties to even, gradual underflow, overflow to infinity).  The
functions below are written from the Rust sources they cite, not from the C oracle and not from numpy.

Two facts are recorded while a function runs (``Trace``):

* ``order_free``: every *accumulated* sum (``sumlx``, ``suml2``, ``sum``, ``slx``, ``sl2``) was exact in any order of
  its terms: all terms are multiples of one power of two ``g`` and the sum of their magnitudes is below
  ``2**24 * g``, so no partial sum of any ordering rounds.  The result then does not depend on the order of the
  summation at all: it follows from the algorithm's definition in rational arithmetic plus single correctly
  rounded operations (a product, a quotient), each of which IEEE-754 fixes uniquely.
* ``inexact``: how many operations rounded at all.  Zero means that the result is the one real arithmetic gives.

``Trace.branches`` collects the names of the branches taken, so that a test can state which case covers which
lines of the reference.
"""
from __future__ import annotations

import struct
from fractions import Fraction

FIN, INF, NAN = 0, 1, 2


def _floor_log2(a: Fraction) -> int:
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    elif Fraction(2) ** (e + 1) <= a:
        e += 1
    return e


def round_to_format(q: Fraction, p: int, emin: int, emax: int):
    """Round the rational q to the binary format with p significand bits: (rounded value or None for overflow, inexact)."""
    if q == 0:
        return Fraction(0), False
    a = abs(q)
    e = max(_floor_log2(a), emin)
    quantum = Fraction(2) ** (e - (p - 1))
    m = a / quantum
    fl = m.numerator // m.denominator
    rem = m - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (fl & 1)):
        fl += 1
    r = fl * quantum
    if r >= Fraction(2) ** (emax + 1):
        return None, True
    return (r if q > 0 else -r), r != a


class Trace:
    def __init__(self):
        self.inexact = 0
        self.order_free = True
        self.branches = set()
        self.tries = 0

    def hit(self, name):
        self.branches.add(name)


_T = Trace()


def new_trace() -> Trace:
    global _T
    _T = Trace()
    return _T


class F32:
    """One IEEE-754 binary32 value."""
    __slots__ = ("q", "neg", "kind")

    def __init__(self, q=Fraction(0), neg=False, kind=FIN):
        self.q, self.neg, self.kind = q, neg, kind

    # ---- construction ----
    @staticmethod
    def of(v) -> "F32":
        """From an int / Fraction / float that is exactly representable (checked)."""
        if isinstance(v, F32):
            return v
        if isinstance(v, float):
            if v != v:
                return F32(kind=NAN)
            if v in (float("inf"), float("-inf")):
                return F32(neg=v < 0, kind=INF)
            neg = struct.pack("<d", v)[7] >= 0x80
            q = Fraction(v)
        else:
            q = Fraction(v)
            neg = q < 0
        r, inexact = round_to_format(q, 24, -126, 127)
        assert r is not None and not inexact, f"{v!r} is not a binary32 value"
        return F32(q, neg)

    @staticmethod
    def from_bits(u: int) -> "F32":
        sign, e, m = u >> 31, (u >> 23) & 0xFF, u & 0x7FFFFF
        if e == 0xFF:
            return F32(neg=bool(sign), kind=NAN if m else INF)
        q = Fraction(m, 1 << 149) if e == 0 else Fraction((1 << 23) | m) * Fraction(2) ** (e - 150)
        return F32(-q if sign else q, bool(sign))

    def bits(self) -> int:
        s = 0x80000000 if self.neg else 0
        if self.kind == NAN:
            return 0x7FC00000
        if self.kind == INF:
            return s | 0x7F800000
        a = abs(self.q)
        if a == 0:
            return s
        e = _floor_log2(a)
        if e < -126:
            m = a / Fraction(2) ** -149
            assert m.denominator == 1
            return s | int(m)
        m = a / Fraction(2) ** (e - 23)
        assert m.denominator == 1
        return s | ((e + 127) << 23) | (int(m) - (1 << 23))

    def to_float(self) -> float:
        return struct.unpack("<f", struct.pack("<I", self.bits()))[0]

    # ---- rounding of an exact result ----
    @staticmethod
    def _rounded(q: Fraction, neg_if_zero: bool) -> "F32":
        if q == 0:
            return F32(Fraction(0), neg_if_zero)
        r, inexact = round_to_format(q, 24, -126, 127)
        if inexact:
            _T.inexact += 1
        if r is None:
            return F32(neg=q < 0, kind=INF)
        if r == 0:  # underflow keeps the sign
            return F32(Fraction(0), q < 0)
        return F32(r, r < 0)

    # ---- arithmetic (one IEEE operation each) ----
    def __neg__(self):
        return F32(-self.q, not self.neg, self.kind)

    def abs(self):
        return F32(abs(self.q), False, self.kind)

    def __add__(self, o):
        o = F32.of(o)
        if self.kind == NAN or o.kind == NAN:
            return F32(kind=NAN)
        if self.kind == INF or o.kind == INF:
            if self.kind == INF and o.kind == INF:
                return F32(neg=self.neg, kind=INF) if self.neg == o.neg else F32(kind=NAN)
            return F32(neg=self.neg if self.kind == INF else o.neg, kind=INF)
        s = self.q + o.q
        if s == 0:  # x + (-x) = +0 in round-to-nearest; (-0) + (-0) = -0
            return F32(Fraction(0), self.neg and o.neg if (self.q == 0 and o.q == 0) else False)
        return F32._rounded(s, False)

    def __sub__(self, o):
        return self + (-F32.of(o))

    def __mul__(self, o):
        o = F32.of(o)
        neg = self.neg != o.neg
        if self.kind == NAN or o.kind == NAN:
            return F32(kind=NAN)
        if self.kind == INF or o.kind == INF:
            if (self.kind == FIN and self.q == 0) or (o.kind == FIN and o.q == 0):
                return F32(kind=NAN)
            return F32(neg=neg, kind=INF)
        return F32._rounded(self.q * o.q, neg)

    def __truediv__(self, o):
        o = F32.of(o)
        neg = self.neg != o.neg
        if self.kind == NAN or o.kind == NAN:
            return F32(kind=NAN)
        if self.kind == INF:
            return F32(kind=NAN) if o.kind == INF else F32(neg=neg, kind=INF)
        if o.kind == INF:
            return F32(Fraction(0), neg)
        if o.q == 0:
            return F32(kind=NAN) if self.q == 0 else F32(neg=neg, kind=INF)
        return F32._rounded(self.q / o.q, neg)

    # ---- IEEE comparisons (-0 == +0; anything with NaN is false) ----
    def _ord(self):
        if self.kind == INF:
            return (1 if not self.neg else -1, Fraction(0))
        return (0, self.q)

    def __lt__(self, o):
        o = F32.of(o)
        return self.kind != NAN and o.kind != NAN and self._ord() < o._ord()

    def __gt__(self, o):
        o = F32.of(o)
        return self.kind != NAN and o.kind != NAN and self._ord() > o._ord()

    def __le__(self, o):
        o = F32.of(o)
        return self.kind != NAN and o.kind != NAN and self._ord() <= o._ord()

    def __eq__(self, o):
        o = F32.of(o)
        return self.kind != NAN and o.kind != NAN and self._ord() == o._ord()

    def __ne__(self, o):
        return not self.__eq__(o)

    __hash__ = None

    def total_key(self):
        """f32::total_cmp as a sortable key: -NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN."""
        u = self.bits()
        return (u ^ 0x80000000) if not (u >> 31) else (~u & 0xFFFFFFFF)

    def __repr__(self):
        return f"F32({self.to_float()!r})"


ZERO = F32()


def rust_max(a: F32, b: F32) -> F32:
    """f32::max: the other operand if one is NaN (of +-0 either may come back; callers only test the result with > 0)."""
    if a.kind == NAN:
        return b
    if b.kind == NAN:
        return a
    return a if a > b else b


def rust_min(a: F32, b: F32) -> F32:
    if a.kind == NAN:
        return b
    if b.kind == NAN:
        return a
    return a if a < b else b


def nearest_int(v: F32) -> int:
    """quantize.rs:566-570: `v.round() as i32`: half away from zero, saturating, NaN -> 0."""
    if v.kind == NAN:
        return 0
    if v.kind == INF:
        return -(2**31) if v.neg else 2**31 - 1
    a = abs(v.q)
    fl = a.numerator // a.denominator
    if a - fl >= Fraction(1, 2):
        fl += 1
    r = -fl if v.q < 0 else fl
    return max(-(2**31), min(2**31 - 1, r))


def clamp(v: int, lo: int, hi: int) -> int:
    return max(lo, min(hi, v))


def f32_to_f16_bits(v: F32) -> int:
    """half::f16::from_f32: IEEE binary16, round to nearest even, overflow to infinity, subnormals kept."""
    s = 0x8000 if v.neg else 0
    if v.kind == NAN:
        return 0x7E00
    if v.kind == INF:
        return s | 0x7C00
    r, _ = round_to_format(v.q, 11, -14, 15)
    if r is None:
        return s | 0x7C00
    a = abs(r)
    if a == 0:
        return s
    e = _floor_log2(a)
    if e < -14:
        return s | int(a / Fraction(2) ** -24)
    return s | ((e + 15) << 10) | (int(a / Fraction(2) ** (e - 10)) - (1 << 10))


def f16_bits_to_f32(h: int) -> F32:
    sign, e, m = h >> 15, (h >> 10) & 0x1F, h & 0x3FF
    if e == 0x1F:
        return F32(neg=bool(sign), kind=NAN if m else INF)
    q = Fraction(m, 1 << 24) if e == 0 else Fraction((1 << 10) | m) * Fraction(2) ** (e - 25)
    return F32(-q if sign else q, bool(sign))


def acc_sum(terms, seed: F32 = ZERO) -> F32:
    """A running binary32 sum in the given order, and the record of whether any order gives the same bits."""
    s = seed
    finite = [t for t in terms if t.kind == FIN]
    if len(finite) != len(terms):
        _T.order_free = False
    else:
        nz = [t.q for t in finite if t.q != 0]
        if nz:
            # the common grid: the largest power of two that divides every term
            g = min(Fraction(1, t.denominator) * (t.numerator & -t.numerator) for t in nz)
            if sum(abs(t) for t in nz) >= (1 << 24) * g:
                _T.order_free = False
    before = _T.inexact
    for t in terms:
        s = s + t
    if _T.inexact != before:
        _T.order_free = False
    return s


# ------------------------------------------------------------------------------------------------
# quantize.rs:583-644
# ------------------------------------------------------------------------------------------------
def make_qkx1_quants(nmax: int, ntry: int, x):
    """Returns (scale, -min) as F32 and the last quants L."""
    n = len(x)
    L = [0] * n
    lo = min(x, key=F32.total_key)   # :588-592
    hi = max(x, key=F32.total_key)   # :593
    if hi == lo:                     # :596
        _T.hit("qkx1:constant")
        return ZERO, ZERO, L
    if lo > ZERO:
        _T.hit("qkx1:min0=0")
    mn = rust_min(lo, ZERO)          # :601
    iscale = F32.of(nmax) / (hi - mn)  # :604
    scale = F32.of(1) / iscale       # :605
    for t in range(ntry):            # :607
        _T.tries = t + 1
        did_change = False
        terms, suml2 = [], 0
        for i in range(n):
            raw = nearest_int(iscale * (x[i] - mn))
            li = clamp(raw, 0, nmax)
            if raw < 0:
                _T.hit("qkx1:clamp_low")
            if raw > nmax:
                _T.hit("qkx1:clamp_high")
            if li != L[i]:
                L[i] = li
                did_change = True
            terms.append((x[i] - mn) * F32.of(li))
            suml2 += li * li
        sumlx = acc_sum(terms)
        if suml2 == 0:               # :622
            _T.hit("qkx1:suml2==0")
            break
        scale = sumlx / F32.of(suml2)  # :625
        s = acc_sum([x[i] - scale * F32.of(L[i]) for i in range(n)], seed=F32(Fraction(0), True))  # :627-632
        mn = s / F32.of(n)           # :634
        if mn > ZERO:                # :635
            _T.hit("qkx1:min>0->0")
            mn = ZERO
        iscale = F32.of(1) / scale   # :638
        if not did_change:           # :639
            _T.hit(f"qkx1:stop_after_try_{t + 1}")
            break
    else:
        _T.hit("qkx1:all_tries_changed")
    return scale, -mn, L             # :643


# ------------------------------------------------------------------------------------------------
# quantize.rs:738-841
# ------------------------------------------------------------------------------------------------
def make_qx_quants(n: int, nmax: int, x, rmse_type: int):
    """Returns (scale as F32, ls with the offset nmax)."""
    ls = [0] * n
    mx, amax = ZERO, ZERO
    for i in range(n):               # :744-750
        ax = x[i].abs()
        if ax > amax:
            amax, mx = ax, x[i]
    if amax == ZERO:                 # :752
        _T.hit("qx:amax==0")
        return ZERO, ls
    _T.hit("qx:max<0" if mx < ZERO else "qx:max>0")
    iscale = -F32.of(nmax) / mx      # :756
    if rmse_type == 0:               # :758-764
        _T.hit("qx:rmse_type==0")
        for i in range(n):
            ls[i] = nmax + clamp(nearest_int(iscale * x[i]), -nmax, nmax - 1)
        return F32.of(1) / iscale, ls
    weighted = rmse_type % 2 == 1

    def wgt(i):
        return x[i] * x[i] if weighted else F32.of(1)

    tx, t2 = [], []
    for i in range(n):               # :770-776
        raw = nearest_int(iscale * x[i])
        l = clamp(raw, -nmax, nmax - 1)
        if raw > nmax - 1:
            _T.hit("qx:clamp_high")
        ls[i] = l + nmax
        w = wgt(i)
        tx.append(w * x[i] * F32.of(l))
        t2.append(w * F32.of(l * l))
    sumlx, suml2 = acc_sum(tx), acc_sum(t2)
    scale = sumlx / suml2            # :778
    best = scale * sumlx             # :779
    for p in range(3):               # :782
        isc = F32.of(1) / scale
        tx, t2, changed = [], [], False
        for i in range(n):
            l = clamp(nearest_int(isc * x[i]), -nmax, nmax - 1)
            if l + nmax != ls[i]:
                changed = True
            w = wgt(i)
            tx.append(w * x[i] * F32.of(l))
            t2.append(w * F32.of(l * l))
        slx, sl2 = acc_sum(tx), acc_sum(t2)
        if not changed:              # :798
            _T.hit(f"qx:rescale{p + 1}:unchanged")
            break
        if sl2 == ZERO:
            _T.hit(f"qx:rescale{p + 1}:sl2==0")
            break
        if slx * slx <= best * sl2:
            _T.hit(f"qx:rescale{p + 1}:rejected")
            if slx * slx == best * sl2:
                _T.hit("qx:rescale:tie_rejected")
            break
        _T.hit(f"qx:rescale{p + 1}:accepted")
        for i in range(n):           # :802-805
            ls[i] = nmax + clamp(nearest_int(isc * x[i]), -nmax, nmax - 1)
        sumlx, suml2 = slx, sl2
        scale = sumlx / suml2
        best = scale * sumlx
    else:
        _T.hit("qx:rescale:three_accepted")
    for sweep in range(5):           # :813
        n_changed = 0
        for i in range(n):
            w = wgt(i)
            l = ls[i] - nmax
            slx = sumlx - w * x[i] * F32.of(l)
            if slx > ZERO:           # :819
                sl2 = suml2 - w * F32.of(l * l)
                new_l = clamp(nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1)
                if new_l != l:
                    slx = slx + w * x[i] * F32.of(new_l)
                    sl2 = sl2 + w * F32.of(new_l * new_l)
                    if sl2 > ZERO and slx * slx * suml2 > sumlx * sumlx * sl2:  # :825
                        _T.hit(f"qx:descent{sweep + 1}:accepted")
                        ls[i] = nmax + new_l
                        sumlx, suml2 = slx, sl2
                        scale = sumlx / suml2
                        n_changed += 1
                    else:
                        _T.hit(f"qx:descent{sweep + 1}:rejected")
            else:
                _T.hit("qx:descent:slx<=0")
                if slx == ZERO:
                    _T.hit("qx:descent:slx==0")
        if n_changed == 0:           # :835
            _T.hit(f"qx:descent:stop_after_sweep_{sweep + 1}")
            break
    else:
        _T.hit("qx:descent:five_sweeps_changed")
    return scale, ls


# ------------------------------------------------------------------------------------------------
# quantize.rs:655-726
# ------------------------------------------------------------------------------------------------
def make_q3_quants(x, nmax: int, do_rmse: bool):
    """Returns (scale as F32, l with the offset nmax)."""
    n = len(x)
    l = [0] * n
    mx, amax = ZERO, ZERO
    for i in range(n):               # :659-667
        ax = x[i].abs()
        if ax > amax:
            amax, mx = ax, x[i]
    if amax == ZERO:                 # :669
        _T.hit("q3:amax==0")
        return ZERO, l
    _T.hit("q3:max<0" if mx < ZERO else "q3:max>0")
    iscale = -F32.of(nmax) / mx      # :673
    if not do_rmse:                  # :720-725
        _T.hit("q3:no_rmse")
        for i in range(n):
            l[i] = clamp(nearest_int(iscale * x[i]), -nmax, nmax - 1) + nmax
        return F32.of(1) / iscale, l
    tx, t2 = [], []
    for i in range(n):               # :678-685
        raw = nearest_int(iscale * x[i])
        li = clamp(raw, -nmax, nmax - 1)
        if raw > nmax - 1:
            _T.hit("q3:clamp_high")
        l[i] = li
        w = x[i] * x[i]
        tx.append(w * x[i] * F32.of(li))
        t2.append(w * F32.of(li * li))
    sumlx, suml2 = acc_sum(tx), acc_sum(t2)
    for sweep in range(5):           # :688
        n_changed = 0
        for i in range(n):
            w = x[i] * x[i]
            slx = sumlx - w * x[i] * F32.of(l[i])
            if slx > ZERO:           # :693
                sl2 = suml2 - w * F32.of(l[i] * l[i])
                new_l = clamp(nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1)
                if new_l != l[i]:
                    slx = slx + w * x[i] * F32.of(new_l)
                    sl2 = sl2 + w * F32.of(new_l * new_l)
                    if sl2 > ZERO and slx * slx * suml2 > sumlx * sumlx * sl2:  # :700
                        _T.hit(f"q3:descent{sweep + 1}:accepted")
                        l[i] = new_l
                        sumlx, suml2 = slx, sl2
                        n_changed += 1
                    else:
                        _T.hit(f"q3:descent{sweep + 1}:rejected")
            else:
                _T.hit("q3:descent:slx<=0")
        if n_changed == 0:           # :709
            _T.hit(f"q3:descent:stop_after_sweep_{sweep + 1}")
            break
    else:
        _T.hit("q3:descent:five_sweeps_changed")
    return sumlx / suml2, [v + nmax for v in l]  # :714-717


# ------------------------------------------------------------------------------------------------
# block quantizers (k_quants.rs); x: 256 F32 values; return the block's bytes
# ------------------------------------------------------------------------------------------------
def _u16le(h):
    return [h & 0xFF, h >> 8]


def get_scale_min_k4(j, q):  # quantize.rs:844-855
    if j < 4:
        return q[j] & 63, q[j + 4] & 63
    return (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4), (q[j + 4] >> 4) | ((q[j] >> 6) << 4)


def _q45k_common(x, nmax):
    """k_quants.rs:895-943 (Q4_K, nmax 15) and :980-1024 (Q5_K, nmax 31): d, dmin, the packed scales and the quants."""
    scales, mins = [], []
    for j in range(8):
        s, m, _ = make_qkx1_quants(nmax, 5, x[32 * j:32 * j + 32])
        scales.append(s)
        mins.append(m)
    max_scale = max_min = ZERO
    for v in scales:                 # fold(0.0, |max, val| val.max(max))
        max_scale = rust_max(v, max_scale)
    for v in mins:
        max_min = rust_max(v, max_min)
    inv_scale = F32.of(63) / max_scale if max_scale > ZERO else ZERO
    inv_min = F32.of(63) / max_min if max_min > ZERO else ZERO
    sc = [0] * 12
    for j in range(8):
        ls = min(nearest_int(inv_scale * scales[j]), 63) & 0xFF
        lm = min(nearest_int(inv_min * mins[j]), 63) & 0xFF
        if j < 4:
            sc[j], sc[j + 4] = ls, lm
        else:
            sc[j + 4] = (ls & 0xF) | ((lm & 0xF) << 4)
            sc[j - 4] |= ((ls >> 4) << 6) & 0xFF
            sc[j] |= ((lm >> 4) << 6) & 0xFF
    d = f32_to_f16_bits(max_scale / F32.of(63))
    dmin = f32_to_f16_bits(max_min / F32.of(63))
    L = [0] * 256
    for j in range(8):
        s6, m6 = get_scale_min_k4(j, sc)
        dq = f16_bits_to_f32(d) * F32.of(s6)
        if dq != ZERO:
            dm = f16_bits_to_f32(dmin) * F32.of(m6)
            for ii in range(32):
                L[32 * j + ii] = clamp(nearest_int((x[32 * j + ii] + dm) / dq), 0, nmax)
    return d, dmin, sc, L


def quantize_q4k_block(x):  # k_quants.rs:876-955
    d, dmin, sc, L = _q45k_common(x, 15)
    qs = [0] * 128
    for j in range(0, 256, 64):
        for l in range(32):
            qs[(j // 64) * 32 + l] = L[j + l] | (L[j + l + 32] << 4)
    return bytes(_u16le(d) + _u16le(dmin) + sc + qs)


def quantize_q5k_block(x):  # k_quants.rs:960-1051
    d, dmin, sc, L = _q45k_common(x, 31)
    qs, qh = [0] * 128, [0] * 32
    m1, m2 = 1, 2
    for n in range(0, 256, 64):
        for j in range(32):
            l1, l2 = L[n + j], L[n + j + 32]
            if l1 > 15:
                l1 -= 16
                qh[j] |= m1
            if l2 > 15:
                l2 -= 16
                qh[j] |= m2
            qs[(n // 64) * 32 + j] = l1 | (l2 << 4)
        m1, m2 = (m1 << 2) & 0xFF, (m2 << 2) & 0xFF
    return bytes(_u16le(d) + _u16le(dmin) + sc + qh + qs)


def quantize_q6k_block(x):  # k_quants.rs:1056-1134
    L = [0] * 256
    scales_f = []
    max_scale = max_abs = ZERO
    for ib in range(16):
        scale, ls = make_qx_quants(16, 32, x[16 * ib:16 * ib + 16], 1)
        L[16 * ib:16 * ib + 16] = ls
        scales_f.append(scale)
        if scale.abs() > max_abs:    # :1090 first strictly greater
            max_abs, max_scale = scale.abs(), scale
    iscale = F32.of(-128) / max_scale
    d = f32_to_f16_bits(F32.of(1) / iscale)
    sc = [min(nearest_int(iscale * s), 127) for s in scales_f]   # `as i8`
    sc = [((v + 128) & 0xFF) - 128 for v in sc]
    for j in range(16):
        dq = f16_bits_to_f32(d) * F32.of(sc[j])
        if dq != ZERO:
            for ii in range(16):
                L[16 * j + ii] = clamp(nearest_int(x[16 * j + ii] / dq), -32, 31) + 32
    ql, qh = [0] * 128, [0] * 64
    for j in range(0, 256, 128):
        for l in range(32):
            q1, q2, q3, q4 = (L[j + l + 32 * g] for g in range(4))
            ql[j // 2 + l] = (q1 & 0xF) | ((q3 & 0xF) << 4)
            ql[j // 2 + l + 32] = (q2 & 0xF) | ((q4 & 0xF) << 4)
            qh[j // 4 + l] = (q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6)
    return bytes(ql + qh + [v & 0xFF for v in sc] + _u16le(d))


def quantize_q3k_block(x):  # k_quants.rs:1139-1237
    scales_f = [make_q3_quants(x[16 * j:16 * j + 16], 4, True)[0] for j in range(16)]
    max_scale = ZERO
    for s in scales_f:               # :1164-1169
        if s.abs() > max_scale.abs():
            max_scale = s
    sc = [0] * 12
    if max_scale != ZERO:
        iscale = F32.of(-32) / max_scale
        for j, s in enumerate(scales_f):
            lv = clamp(nearest_int(iscale * s), -32, 31) + 32
            if j < 8:
                sc[j] = lv & 0xF
            else:
                sc[j - 8] |= (lv & 0xF) << 4
            sc[j % 4 + 8] |= ((lv >> 4) << (2 * (j // 4))) & 0xFF
        d = f32_to_f16_bits(F32.of(1) / iscale)
    else:
        d = 0
    L = [0] * 256
    for j in range(16):
        s4 = sc[j] & 0xF if j < 8 else sc[j - 8] >> 4
        s6 = (s4 | (((sc[8 + j % 4] >> (2 * (j // 4))) & 3) << 4)) - 32
        dq = f16_bits_to_f32(d) * F32.of(s6)
        if dq != ZERO:
            for ii in range(16):
                L[16 * j + ii] = clamp(nearest_int(x[16 * j + ii] / dq), -4, 3) + 4
    hmask = [0] * 32
    m, hm = 0, 1
    for i in range(256):             # :1213-1223
        if L[i] > 3:
            hmask[m] |= hm
            L[i] -= 4
        m += 1
        if m == 32:
            m, hm = 0, (hm << 1) & 0xFF
    qs = [0] * 64
    for j in range(0, 256, 128):
        for l in range(32):
            qs[j // 4 + l] = L[j + l] | (L[j + l + 32] << 2) | (L[j + l + 64] << 4) | (L[j + l + 96] << 6)
    return bytes(hmask + qs + sc + _u16le(d))


def quantize_q2k_block(x):  # k_quants.rs:1242-1323
    scales, mins = [], []
    for j in range(16):
        s, m, _ = make_qkx1_quants(3, 5, x[16 * j:16 * j + 16])
        scales.append(s)
        mins.append(m)
    max_scale = max_min = ZERO
    for v in scales:
        max_scale = rust_max(v, max_scale)
    for v in mins:
        max_min = rust_max(v, max_min)
    sc = [0] * 16
    if max_scale > ZERO:
        iscale = F32.of(15) / max_scale
        for j in range(16):
            sc[j] = nearest_int(iscale * scales[j]) & 0xFF
        d = f32_to_f16_bits(max_scale / F32.of(15))
    else:
        d = 0
    if max_min > ZERO:
        iscale = F32.of(15) / max_min
        for j in range(16):
            sc[j] |= ((nearest_int(iscale * mins[j]) & 0xFF) << 4) & 0xFF
        dmin = f32_to_f16_bits(max_min / F32.of(15))
    else:
        dmin = 0
    L = [0] * 256
    for j in range(16):
        dq = f16_bits_to_f32(d) * F32.of(sc[j] & 0xF)
        if dq == ZERO:
            continue
        dm = f16_bits_to_f32(dmin) * F32.of(sc[j] >> 4)
        for ii in range(16):
            L[16 * j + ii] = clamp(nearest_int((x[16 * j + ii] + dm) / dq), 0, 3)
    qs = [0] * 64
    for j in range(0, 256, 128):
        for l in range(32):
            qs[j // 4 + l] = L[j + l] | (L[j + l + 32] << 2) | (L[j + l + 64] << 4) | (L[j + l + 96] << 6)
    return bytes(sc + qs + _u16le(d) + _u16le(dmin))


BLOCK_QUANTIZERS = {12: quantize_q4k_block, 13: quantize_q5k_block, 14: quantize_q6k_block,
                    11: quantize_q3k_block, 10: quantize_q2k_block}


# ------------------------------------------------------------------------------------------------
# whole tensors: a trailing partial super-block is emitted as zeros (k_quants.rs:890-892, :1070-1072)
# ------------------------------------------------------------------------------------------------
BLOCK_BYTES = {12: 144, 13: 176, 14: 210, 11: 110, 10: 84}


def quantize_tensor(t: int, x) -> bytes:
    if t == 8:
        return quantize_q8_0(x)
    out = b""
    for b in range((len(x) + 255) // 256):
        blk = x[256 * b:256 * b + 256]
        out += BLOCK_QUANTIZERS[t](blk) if len(blk) == 256 else bytes(BLOCK_BYTES[t])
    return out


def quantize_q8_0(x) -> bytes:  # quantize.rs:268-300
    out = []
    for b in range((len(x) + 31) // 32):
        blk = x[32 * b:32 * b + 32]
        amax = ZERO
        for v in blk:                # fold(0.0, |acc, x| acc.max(x.abs()))
            amax = rust_max(amax, v.abs())
        scale = amax / F32.of(127)
        iscale = ZERO if amax == ZERO else F32.of(127) / amax
        out += _u16le(f32_to_f16_bits(scale))
        for i in range(32):
            out.append(clamp(nearest_int(blk[i] * iscale), -127, 127) & 0xFF if i < len(blk) else 0)
    return bytes(out)


# ------------------------------------------------------------------------------------------------
# dequantizers: every product and difference is rounded on its own
# ------------------------------------------------------------------------------------------------
def dequantize_q8_0(raw: bytes, n: int):  # dequant.rs:466-495
    y = []
    for b in range(len(raw) // 34):
        blk = raw[34 * b:34 * b + 34]
        scale = f16_bits_to_f32(blk[0] | (blk[1] << 8))
        for i in range(32):
            q = blk[2 + i] - 256 if blk[2 + i] >= 128 else blk[2 + i]
            y.append(F32.of(q) * scale)
    return y[:n]


def dequantize_q4k(raw: bytes, n: int, ggml_order: bool = False):
    """k_quants.rs:358-404 (the reference's order).  ggml_order: the inverse of quantize_q4k's packing (:946-951) instead."""
    y = []
    for b in range(len(raw) // 144):
        blk = raw[144 * b:144 * b + 144]
        d, dmin = f16_bits_to_f32(blk[0] | (blk[1] << 8)), f16_bits_to_f32(blk[2] | (blk[3] << 8))
        sc, qs = list(blk[4:16]), blk[16:]
        is_ = 0
        for j in range(0, 256, 64):
            s1, m1 = get_scale_min_k4(is_, sc)
            s2, m2 = get_scale_min_k4(is_ + 1, sc)
            d1, dm1 = d * F32.of(s1), dmin * F32.of(m1)
            d2, dm2 = d * F32.of(s2), dmin * F32.of(m2)
            q = qs[j // 2:j // 2 + 32]
            if ggml_order:
                y += [d1 * F32.of(q[l] & 0xF) - dm1 for l in range(32)]
                y += [d2 * F32.of(q[l] >> 4) - dm2 for l in range(32)]
            else:
                y += [d1 * F32.of(q[l] & 0xF) - dm1 for l in range(16)]
                y += [d1 * F32.of(q[l] >> 4) - dm1 for l in range(16)]
                y += [d2 * F32.of(q[16 + l] & 0xF) - dm2 for l in range(16)]
                y += [d2 * F32.of(q[16 + l] >> 4) - dm2 for l in range(16)]
            is_ += 2
    return y[:n]


def dequantize_q6k(raw: bytes, n: int):  # k_quants.rs:474-496
    y = []
    for b in range(len(raw) // 210):
        blk = raw[210 * b:210 * b + 210]
        d = f16_bits_to_f32(blk[208] | (blk[209] << 8))
        out = [None] * 256
        for c in range(2):
            ql, qh = blk[64 * c:], blk[128 + 32 * c:]
            sc = [v - 256 if v >= 128 else v for v in blk[192 + 8 * c:192 + 8 * c + 8]]
            for l in range(32):
                is_ = l // 16
                q1 = ((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32
                q2 = ((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32
                q3 = ((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32
                q4 = ((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32
                out[128 * c + l] = d * F32.of(sc[is_]) * F32.of(q1)
                out[128 * c + l + 32] = d * F32.of(sc[is_ + 2]) * F32.of(q2)
                out[128 * c + l + 64] = d * F32.of(sc[is_ + 4]) * F32.of(q3)
                out[128 * c + l + 96] = d * F32.of(sc[is_ + 6]) * F32.of(q4)
        y += out
    return y[:n]
