"""Host-side check of the range test that admits the short requantization form of the kernels.

The kernels (short_ok in esp-dl_amd/csrc/mbconv_s8_stages.h, the same test spelled out in the dense and
depthwise kernels) take the short form for a channel when 1 <= s <= 31 and
|bias + 2^(s-1)| + K * 2^14 < 2^(31 - max(0, 8 - s)).  The short form starts the int32 accumulator at
bias + 2^(s-1), shifts left by max(0, 8 - s) and right by max(0, s - 8), saturates to int16 and keeps the high
byte.  Here that arithmetic is replayed with 32-bit wrap-around on accumulators at and around the bound and
compared with shift_and_round in exact integers (esp-dl/dl/tool/src/dl_tool.cpp:121-136): inside the bound the
two agree for every sum the reduction can reach; just outside it there are sums for which they differ, i.e. the
bound is not merely sufficient by a wide margin."""
import numpy as np


def short_ok(s, bias, mac_bound):
    if s < 1 or s > 31:
        return False
    lim = 1 << (31 - max(0, 8 - s))
    return abs(bias + (1 << (s - 1))) + mac_bound < lim


def wrap32(v):
    return (v + (1 << 31)) % (1 << 32) - (1 << 31)


def short_form(sum_, bias, s, relu=False):
    acc = wrap32(bias + (1 << (s - 1)) + sum_)  # what the int32 accumulator holds
    t = wrap32(acc << max(0, 8 - s)) >> max(0, s - 8)
    t = max(-32768, min(32767, t))  # v_cvt_pk_i16_i32
    if relu:
        t = max(t, 0)
    return t >> 8  # the high byte


def exact(sum_, bias, s, relu=False):
    q = (sum_ + bias + (1 << (s - 1))) >> s  # floor((v + 2^(s-1)) / 2^s) in unbounded integers
    if relu:
        q = max(q, 0)
    return max(-128, min(127, q))


def test_short_form_is_exact_inside_the_bound():
    rng = np.random.default_rng(5)
    for k_total in (9, 24, 576, 1280, 2304, 16384):
        mac = k_total * 16384
        for s in range(1, 32):
            biases = [0, 1, -1, 4096, -4096, 1 << 20, -(1 << 20), (1 << 30) - 1, -((1 << 30) - 1)]
            # the largest bias magnitudes the test still admits for this shift
            lim = (1 << (31 - max(0, 8 - s))) - mac - (1 << (s - 1))
            if lim > 1:
                biases += [lim - 1, -(lim - 1) + (1 << s)]
            for bias in biases:
                if not short_ok(s, bias, mac):
                    continue
                sums = [mac, -mac, mac - 1, -mac + 1, 0, 1, -1]
                sums += [int(v) for v in rng.integers(-mac, mac + 1, size=40)]
                # sums that put v + 2^(s-1) on and next to multiples of 2^s (ties of the rounding)
                for q in (-130, -129, -128, -1, 0, 1, 126, 127, 128):
                    base = q * (1 << s) - bias - (1 << (s - 1))
                    sums += [base - 1, base, base + 1]
                for sm in sums:
                    if abs(sm) > mac:
                        continue
                    for relu in (False, True):
                        assert short_form(sm, bias, s, relu) == exact(sm, bias, s, relu), (k_total, s, bias, sm, relu)


def test_bound_is_tight():
    """Outside the bound the short form does go wrong for some reachable sum: the range test is needed."""
    found = 0
    for k_total in (576, 2304):
        mac = k_total * 16384
        for s in (1, 4, 7, 8, 24, 31):
            lim = (1 << (31 - max(0, 8 - s)))
            bias = lim - (1 << (s - 1))  # start value at the limit: any positive sum overflows
            assert not short_ok(s, bias, mac)
            if any(short_form(sm, bias, s) != exact(sm, bias, s) for sm in (mac, mac // 2, 1 << 14, 1)):
                found += 1
    assert found >= 6
