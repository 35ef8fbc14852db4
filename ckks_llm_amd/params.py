"""Prime sets: the benchmark configurations and the reference's own parameter sets (Params.cuh)."""

# config 1: 4 largest primes < 2^36 with q = 1 mod 2^13
CFG1_Q = [0xffffee001, 0xffffc4001, 0xffffbe001, 0xffffba001]
# config 2: 24 largest primes < 2^36 with q = 1 mod 2^17 (the commented 36-bit set of Params.cuh:96-106)
CFG2_Q = [0xffff00001, 0xfff9c0001, 0xfff8e0001, 0xfff840001, 0xfff700001, 0xfff640001,
          0xfff4c0001, 0xfff3c0001, 0xfff280001, 0xfff100001, 0xffefe0001, 0xffee80001,
          0xffee20001, 0xffeda0001, 0xffeca0001, 0xffea40001, 0xffe940001, 0xffe920001,
          0xffe760001, 0xffe040001, 0xffdf80001, 0xffdf00001, 0xffdd20001, 0xffdbc0001]
# config 3: 6 largest primes < 2^37 with p = 1 mod 2^17
CFG3_P = [0x1ffffe0001, 0x1ffffc0001, 0x1fffea0001, 0x1fffb60001, 0x1fffaa0001, 0x1fff8c0001]

# Params.cuh:17-33 (logN = 13), :36-60 (14), :62-86 (15), :88-171 (16)
REF_PARAMS = {
    13: dict(q=[0x4001b00001, 0xfff9c0001, 0xfff8e0001, 0xfff840001, 0xfff700001],
             p=[0x10a19000001],
             t=[0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001], gamma=3),
    14: dict(q=[0x4001b00001, 0xfff9c0001, 0xfff8e0001, 0xfff840001, 0xfff700001, 0xfff640001,
                0x1000a20001, 0x1000b40001, 0x1000f60001, 0x10011a0001],
             p=[0x10a19000001, 0x10a3b000001],
             t=[0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001, 0xfffffffff5a0001], gamma=3),
    15: dict(q=[0x20000018e0001, 0x2000001c00001, 0x2000001ca0001, 0x2000001d20001,
                0x1fffffee80001, 0x1fffffede0001, 0x1fffffec40001, 0x1fffffe780001,
                0x2000000ce0001, 0x20000013a0001, 0x20000013c0001, 0x20000015a0001],
             p=[0x2000002600001, 0x20000027e0001, 0x2000002800001, 0x20000029e0001],
             t=[0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001, 0xfffffffff5a0001,
                0xfffffffff2a0001, 0xfffffffff240001, 0xffffffffefe0001], gamma=4),
    16: dict(q=[0x20000018e0001, 0x2000001c00001, 0x2000001ca0001, 0x2000001d20001,
                0x1fffffee80001, 0x1fffffede0001, 0x1fffffec40001, 0x1fffffe780001,
                0x2000000ce0001, 0x20000013a0001, 0x20000013c0001, 0x20000015a0001,
                0x1ffffffea0001, 0x1ffffffd40001, 0x1ffffffba0001, 0x1ffffffb40001,
                0x20000001a0001, 0x20000005e0001, 0x2000000860001, 0x2000000b00001,
                0x1ffffffb00001, 0x1ffffffa20001, 0x1ffffff780001, 0x1ffffff5c0001,
                0x1fffffe5a0001, 0x1fffffe480001, 0x1fffffde80001, 0x1fffffde20001],
             p=[0x2000002600001, 0x20000027e0001, 0x2000002800001, 0x20000029e0001],
             t=[0xffffffffffc0001, 0xfffffffff840001, 0xfffffffff6a0001, 0xfffffffff5a0001,
                0xfffffffff2a0001, 0xfffffffff240001, 0xffffffffefe0001, 0xffffffffeca0001], gamma=4),
}


def small_primes(bits, two_n, count, skip=0):
    """`count` largest primes below 2**bits with p = 1 (mod two_n); plain trial division / Miller-Rabin via sympy."""
    from sympy import isprime
    out, c = [], (1 << bits) - ((1 << bits) - 1) % two_n
    while len(out) < count + skip:
        if c < (1 << bits) and isprime(c):
            out.append(c)
        c -= two_n
    return out[skip:]
