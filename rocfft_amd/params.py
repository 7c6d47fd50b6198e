"""Transform parameters in the reference clients' vocabulary, and their token strings.

The reference's test and benchmark clients describe a transform with an
`fft_params` object whose `token()` names the case
(shared/fft_params.h:726-900, e.g.
`real_forward_len_65536_single_op_batch_4096_istride_1_R_ostride_1_HI_idist_65536_odist_32769_ioffset_0_0_ooffset_0_0`)
and whose `from_token()` reads it back (:901-1059).  `FFTParams` is the same
surface over this library's ctypes binding, so that existing token lists and
perf scripts can drive it: lengths and strides are ROW-major here (slowest
dimension first, as in the tokens), and are reversed when the plan is created,
because `rocfft_plan_create` takes the fastest dimension first
(include/rocfft/rocfft.h).

Nothing here computes a transform; `make_plan` raises if the library is missing.
"""
from . import binding as B

_TYPE_NAMES = {B.COMPLEX_INTERLEAVED: "CI", B.COMPLEX_PLANAR: "CP", B.REAL: "R",
               B.HERMITIAN_INTERLEAVED: "HI", B.HERMITIAN_PLANAR: "HP"}
_TYPE_VALUES = {v: k for k, v in _TYPE_NAMES.items()}
_KIND_NAMES = {B.COMPLEX_FORWARD: "complex_forward", B.COMPLEX_INVERSE: "complex_inverse",
               B.REAL_FORWARD: "real_forward", B.REAL_INVERSE: "real_inverse"}
_PRECISION_NAMES = {B.SINGLE: "single", B.DOUBLE: "double", B.HALF: "half"}
# the factor from_token() assigns to a token that ends in "_scale" (fft_params.h:1046-1051)
TOKEN_SCALE_FACTOR = 0.1239


class TokenError(ValueError):
    pass


def _prod(values):
    p = 1
    for v in values:
        p *= int(v)
    return p


def _contiguous(lengths):
    """row-major unit-stride strides of an array with these lengths"""
    strides = [1] * len(lengths)
    for i in range(len(lengths) - 2, -1, -1):
        strides[i] = strides[i + 1] * lengths[i + 1]
    return strides


class FFTParams:
    def __init__(self, transform_type=B.COMPLEX_FORWARD, length=(), precision=B.SINGLE,
                 placement=B.INPLACE, nbatch=1, istride=None, ostride=None, idist=0, odist=0,
                 ioffset=None, ooffset=None, itype=None, otype=None, scale_factor=1.0):
        self.transform_type = transform_type
        self.length = [int(v) for v in length]
        self.precision = precision
        self.placement = placement
        self.nbatch = int(nbatch)
        self.istride = list(istride) if istride else []
        self.ostride = list(ostride) if ostride else []
        self.idist = int(idist)
        self.odist = int(odist)
        self.ioffset = list(ioffset) if ioffset else [0, 0]
        self.ooffset = list(ooffset) if ooffset else [0, 0]
        self.itype = itype
        self.otype = otype
        self.scale_factor = float(scale_factor)

    # ------------------------------------------------------------------ derived sizes
    def dim(self):
        return len(self.length)

    def ilength(self):
        n = list(self.length)
        if self.transform_type == B.REAL_INVERSE:
            n[-1] = n[-1] // 2 + 1
        return n

    def olength(self):
        n = list(self.length)
        if self.transform_type == B.REAL_FORWARD:
            n[-1] = n[-1] // 2 + 1
        return n

    def validate(self):
        """Fills in whatever was left unset with the reference clients' defaults: array types
        from the transform type, unit-stride row-major strides, distances that pack the
        batches, and for in-place real transforms the padded real rows of 2(N/2+1) values."""
        real_fwd = self.transform_type == B.REAL_FORWARD
        real_inv = self.transform_type == B.REAL_INVERSE
        if self.itype is None:
            self.itype = B.REAL if real_fwd else B.HERMITIAN_INTERLEAVED if real_inv \
                else B.COMPLEX_INTERLEAVED
        if self.otype is None:
            self.otype = B.HERMITIAN_INTERLEAVED if real_fwd else B.REAL if real_inv \
                else B.COMPLEX_INTERLEAVED
        if not self.length or any(v < 1 for v in self.length) or self.dim() > 3:
            raise TokenError("1 to 3 positive lengths are needed")
        inplace = self.placement == B.INPLACE
        padded = list(self.length)
        padded[-1] = 2 * (self.length[-1] // 2 + 1)

        def fill(strides, dist, lengths, is_real):
            base = padded if (inplace and is_real) else lengths
            if not strides:
                strides = _contiguous(base)
            if not dist:
                if len(strides) == len(lengths) and strides == _contiguous(base):
                    dist = _prod(base)
                else:
                    dist = max(s * n for s, n in zip(strides, lengths))
            return strides, dist

        self.istride, self.idist = fill(self.istride, self.idist, self.ilength(), real_fwd)
        self.ostride, self.odist = fill(self.ostride, self.odist, self.olength(), real_inv)
        if len(self.istride) != self.dim() or len(self.ostride) != self.dim():
            raise TokenError("one stride per dimension is needed")
        return self

    # ------------------------------------------------------------------ token
    def token(self):
        p = self
        out = _KIND_NAMES[p.transform_type] + "_len"
        out += "".join("_%d" % v for v in p.length)
        out += "_%s_" % _PRECISION_NAMES[p.precision]
        out += "ip_" if p.placement == B.INPLACE else "op_"
        out += "batch_%d" % p.nbatch
        out += "_istride" + "".join("_%d" % v for v in p.istride) + "_" + _TYPE_NAMES.get(p.itype, "UN")
        out += "_ostride" + "".join("_%d" % v for v in p.ostride) + "_" + _TYPE_NAMES.get(p.otype, "UN")
        out += "_idist_%d_odist_%d" % (p.idist, p.odist)
        out += "_ioffset" + "".join("_%d" % v for v in p.ioffset)
        out += "_ooffset" + "".join("_%d" % v for v in p.ooffset)
        if p.scale_factor != 1.0:
            out += "_scale"
        return out

    @classmethod
    def from_token(cls, token):
        vals = token.split("_")
        pos = [0]

        def take():
            if pos[0] >= len(vals):
                raise TokenError("token ends early: " + token)
            v = vals[pos[0]]
            pos[0] += 1
            return v

        def numbers(word):
            if take() != word:
                raise TokenError("expected '%s' in %s" % (word, token))
            out = []
            while pos[0] < len(vals) and vals[pos[0]].isdigit():
                out.append(int(take()))
            return out

        def number(word):
            v = numbers(word)
            if len(v) != 1:
                raise TokenError("expected one number after '%s' in %s" % (word, token))
            return v[0]

        domain, direction = take(), take()
        if domain not in ("complex", "real") or direction not in ("forward", "inverse"):
            raise TokenError("unknown transform type in " + token)
        kind = {("complex", "forward"): B.COMPLEX_FORWARD, ("complex", "inverse"): B.COMPLEX_INVERSE,
                ("real", "forward"): B.REAL_FORWARD, ("real", "inverse"): B.REAL_INVERSE}[(domain, direction)]
        p = cls(kind)
        p.length = numbers("len")
        prec = take()
        if prec not in ("single", "double", "half"):
            raise TokenError("unknown precision in " + token)
        p.precision = {"single": B.SINGLE, "double": B.DOUBLE, "half": B.HALF}[prec]
        place = take()
        if place not in ("ip", "op"):
            raise TokenError("unknown placement in " + token)
        p.placement = B.INPLACE if place == "ip" else B.NOTINPLACE
        p.nbatch = number("batch")
        while pos[0] < len(vals):
            word = vals[pos[0]]
            if word == "istride":
                p.istride = numbers("istride")
                p.itype = _TYPE_VALUES.get(take())
            elif word == "ostride":
                p.ostride = numbers("ostride")
                p.otype = _TYPE_VALUES.get(take())
            elif word == "idist":
                p.idist = number("idist")
            elif word == "odist":
                p.odist = number("odist")
            elif word == "ioffset":
                p.ioffset = (numbers("ioffset") + [0, 0])[:2]
            elif word == "ooffset":
                p.ooffset = (numbers("ooffset") + [0, 0])[:2]
            elif word in ("ifield", "ofield", "multiGPU", "multigpu"):
                raise TokenError("fields, bricks and several GPUs are not supported: " + token)
            elif word == "CB":
                raise TokenError("load/store callbacks are not supported: " + token)
            elif word == "scale":
                p.scale_factor = TOKEN_SCALE_FACTOR
                pos[0] += 1
            else:
                raise TokenError("unexpected '%s' in %s" % (word, token))
        return p

    # ------------------------------------------------------------------ buffers and plan
    def _extent(self, lengths, strides, dist, offset):
        return offset + (self.nbatch - 1) * dist + sum((n - 1) * s for n, s in zip(lengths, strides)) + 1

    def isize(self):
        """elements (of the input array type) every input buffer must hold"""
        return self._extent(self.ilength(), self.istride, self.idist, max(self.ioffset))

    def osize(self):
        return self._extent(self.olength(), self.ostride, self.odist, max(self.ooffset))

    def ibuffers(self):
        return 2 if self.itype in (B.COMPLEX_PLANAR, B.HERMITIAN_PLANAR) else 1

    def obuffers(self):
        return 2 if self.otype in (B.COMPLEX_PLANAR, B.HERMITIAN_PLANAR) else 1

    def make_plan(self, lib=None):
        """rocfft_plan_description_create -> set_data_layout -> [set_scale_factor] -> rocfft_plan_create,
        the call order of the reference clients (shared/rocfft_params.h:341-470)."""
        self.validate()
        desc = B.PlanDescription(lib)
        desc.set_data_layout(self.itype, self.otype, self.ioffset, self.ooffset,
                             list(reversed(self.istride)), self.idist, list(reversed(self.ostride)),
                             self.odist)
        if self.scale_factor != 1.0:
            desc.set_scale_factor(self.scale_factor)
        return B.Plan(self.placement, self.transform_type, self.precision, list(reversed(self.length)),
                      self.nbatch, desc, lib=lib)

    def opscount(self):
        """the operation count rocfft-bench divides by the time: 5 N log2 N per complex
        transform, 2.5 N log2 N per real one (clients/bench/bench.cpp:468-476)"""
        import math
        total = _prod(self.length)
        k = 2.5 if self.transform_type in (B.REAL_FORWARD, B.REAL_INVERSE) else 5.0
        return self.nbatch * k * total * math.log2(total) if total > 1 else 0.0
