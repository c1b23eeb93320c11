"""The uniform number of one draw: a function of (seed, request, step) and nothing
else, so that what a request draws does not depend on which other requests share
its batch.  Integer mixing (three rounds of the splitmix64 finaliser, one each for seed, request
and step), top 24 bits
taken as a float32 in [0, 1)."""

_M = (1 << 64) - 1


def _mix(x):
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9 & _M
    x = (x ^ (x >> 27)) * 0x94D049BB133111EB & _M
    return x ^ (x >> 31)


def uniform(seed, request, step):
    x = _mix((seed & _M) + 0x9E3779B97F4A7C15 & _M)
    x = _mix((x ^ (request & _M)) + 0x9E3779B97F4A7C15 & _M)
    x = _mix((x ^ (step & _M)) + 0x9E3779B97F4A7C15 & _M)
    return (x >> 40) / float(1 << 24)
