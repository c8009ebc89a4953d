"""Big-integer model of Goldilocks and its quadratic extension X^2 = 7, plus
definitions-first (brute force) versions of the objects the sumcheck path
manipulates.  Written against the mathematics only; shares no code with the C
checker or the GPU library, which are both tested against it."""
import random

P = 2**64 - 2**32 + 1
W = 7


def from_i64(x):
    return x % P


class E2:
    __slots__ = ("a", "b")

    def __init__(self, a=0, b=0):
        self.a, self.b = a % P, b % P

    def __add__(self, o):
        o = lift(o)
        return E2(self.a + o.a, self.b + o.b)

    __radd__ = __add__

    def __sub__(self, o):
        o = lift(o)
        return E2(self.a - o.a, self.b - o.b)

    def __rsub__(self, o):
        return lift(o) - self

    def __neg__(self):
        return E2(-self.a, -self.b)

    def __mul__(self, o):
        o = lift(o)
        return E2(self.a * o.a + W * self.b * o.b, self.a * o.b + self.b * o.a)

    __rmul__ = __mul__

    def inv(self):
        n = pow((self.a * self.a - W * self.b * self.b) % P, P - 2, P)
        return E2(self.a * n, -self.b * n)

    def __eq__(self, o):
        o = lift(o)
        return self.a == o.a and self.b == o.b

    def __hash__(self):
        return hash((self.a, self.b))

    def __repr__(self):
        return f"E2({self.a}, {self.b})"

    def pair(self):
        return (self.a, self.b)


def lift(x):
    return x if isinstance(x, E2) else E2(int(x), 0)


def rand_e2(rng: random.Random):
    return E2(rng.randrange(P), rng.randrange(P))


def eq_at(point, index):
    """eq(point, bits_le(index)) from the definition."""
    acc = E2(1)
    for j, r in enumerate(point):
        acc = acc * (r if (index >> j) & 1 else (1 - r))
    return acc


def mle_eval(values, point):
    """Multilinear extension of `values` (little-endian index) at `point`, from the definition."""
    assert len(values) == 1 << len(point)
    acc = E2(0)
    for i, v in enumerate(values):
        acc = acc + lift(v) * eq_at(point, i)
    return acc


def round_poly_bruteforce(tables, nvars, n, terms, prefix, degree):
    """p_j(t) for j = len(prefix)+1 from the definition of the sumcheck message:
    sum over boolean suffixes x of expr(MLE_k(prefix, t, x)).  A table with m < n
    variables depends on the LAST m variables only."""
    j = len(prefix)
    out = []
    for t in range(degree + 1):
        total = E2(0)
        for x in range(1 << (n - j - 1)):
            full = list(prefix) + [E2(t)] + [E2((x >> b) & 1) for b in range(n - j - 1)]
            vals = []
            for tab, m in zip(tables, nvars):
                vals.append(mle_eval(tab, full[n - m:]))
            for coeff, factors in terms:
                prod = lift(coeff)
                for f in factors:
                    prod = prod * vals[f]
                total = total + prod
        out.append(total)
    return out


def interpolate(evals, r):
    d = len(evals) - 1
    acc = E2(0)
    for k in range(d + 1):
        num, den = E2(1), 1
        for m in range(d + 1):
            if m != k:
                num = num * (r - m)
                den = den * (k - m) % P
        acc = acc + num * pow(den, P - 2, P) * evals[k]
    return acc
