"""The elementwise functions of the package, built from the kernel entry points
(registrations of dpnp/tensor/_elementwise_funcs.py for the ops this library implements)."""
from . import _tensor_elementwise_impl as tei
from ._elementwise_common import BinaryElementwiseFunc, UnaryElementwiseFunc
from ._type_utils import (
    _acceptance_fn_divide,
    _acceptance_fn_negative,
    _acceptance_fn_reciprocal,
    _acceptance_fn_subtract,
    _resolve_weak_types_all_py_ints,
)


def _unary(name, doc, **kw):
    return UnaryElementwiseFunc(name, getattr(tei, f"_{name}_result_type"), getattr(tei, f"_{name}"),
                                doc, **kw)


def _binary(name, doc, inplace=True, **kw):
    return BinaryElementwiseFunc(
        name, getattr(tei, f"_{name}_result_type"), getattr(tei, f"_{name}"), doc,
        binary_inplace_fn=getattr(tei, f"_{name}_inplace") if inplace else None, **kw)


abs = _unary("abs", "abs(x, /, *, out=None, order='K'): elementwise absolute value.")  # noqa: A001
negative = _unary("negative", "Elementwise numerical negative.", acceptance_fn=_acceptance_fn_negative)
positive = _unary("positive", "Elementwise numerical positive.")
square = _unary("square", "Elementwise square.")
sqrt = _unary("sqrt", "Elementwise non-negative square root.")
exp = _unary("exp", "Elementwise exponential.")
log = _unary("log", "Elementwise natural logarithm.")
erf = _unary("erf", "Elementwise error function.")
sin = _unary("sin", "Elementwise sine.")
cos = _unary("cos", "Elementwise cosine.")
tan = _unary("tan", "Elementwise tangent.")
tanh = _unary("tanh", "Elementwise hyperbolic tangent.")
exp2 = _unary("exp2", "Elementwise 2**x.")
expm1 = _unary("expm1", "Elementwise exp(x) - 1.")
log2 = _unary("log2", "Elementwise base-2 logarithm.")
log10 = _unary("log10", "Elementwise base-10 logarithm.")
log1p = _unary("log1p", "Elementwise log(1 + x).")
rsqrt = _unary("rsqrt", "Elementwise reciprocal square root.")
cbrt = _unary("cbrt", "Elementwise cube root.")
reciprocal = _unary("reciprocal", "Elementwise 1/x.", acceptance_fn=_acceptance_fn_reciprocal)
floor = _unary("floor", "Elementwise floor.")
ceil = _unary("ceil", "Elementwise ceiling.")
trunc = _unary("trunc", "Elementwise truncation.")
sign = _unary("sign", "Elementwise sign.")
isnan = _unary("isnan", "Elementwise test for NaN.")
isinf = _unary("isinf", "Elementwise test for infinity.")
isfinite = _unary("isfinite", "Elementwise test for finiteness.")
logical_not = _unary("logical_not", "Elementwise logical negation.")
bitwise_invert = _unary("bitwise_invert", "Elementwise bit inversion.")
signbit = _unary("signbit", "Elementwise test of the sign bit.")
asin = _unary("asin", "Elementwise inverse sine.")
acos = _unary("acos", "Elementwise inverse cosine.")
atan = _unary("atan", "Elementwise inverse tangent.")
sinh = _unary("sinh", "Elementwise hyperbolic sine.")
cosh = _unary("cosh", "Elementwise hyperbolic cosine.")
asinh = _unary("asinh", "Elementwise inverse hyperbolic sine.")
acosh = _unary("acosh", "Elementwise inverse hyperbolic cosine.")
atanh = _unary("atanh", "Elementwise inverse hyperbolic tangent.")
round = _unary("round", "Elementwise rounding to the nearest integer, ties to even.")  # noqa: A001
conj = _unary("conj", "Elementwise complex conjugate.")
real = _unary("real", "Elementwise real part.")
imag = _unary("imag", "Elementwise imaginary part.")
proj = _unary("proj", "Elementwise projection onto the Riemann sphere.")
angle = _unary("angle", "Elementwise argument of a complex number.")

add = _binary("add", "add(x1, x2, /, *, out=None, order='K'): elementwise sum.")
subtract = _binary("subtract", "Elementwise difference.", acceptance_fn=_acceptance_fn_subtract)
multiply = _binary("multiply", "Elementwise product.")
divide = _binary("divide", "Elementwise true division.", acceptance_fn=_acceptance_fn_divide,
                 weak_type_resolver=_resolve_weak_types_all_py_ints)
bitwise_and = _binary("bitwise_and", "Elementwise bitwise and (logical for bool).")
bitwise_or = _binary("bitwise_or", "Elementwise bitwise or (logical for bool).")
bitwise_xor = _binary("bitwise_xor", "Elementwise bitwise xor (logical for bool).")
_cmp = dict(inplace=False, weak_type_resolver=_resolve_weak_types_all_py_ints)
equal = _binary("equal", "Elementwise x1 == x2.", **_cmp)
not_equal = _binary("not_equal", "Elementwise x1 != x2.", **_cmp)
less = _binary("less", "Elementwise x1 < x2.", **_cmp)
less_equal = _binary("less_equal", "Elementwise x1 <= x2.", **_cmp)
greater = _binary("greater", "Elementwise x1 > x2.", **_cmp)
greater_equal = _binary("greater_equal", "Elementwise x1 >= x2.", **_cmp)
maximum = _binary("maximum", "Elementwise maximum, NaN propagating.")
minimum = _binary("minimum", "Elementwise minimum, NaN propagating.")
logical_and = _binary("logical_and", "Elementwise logical and.", inplace=False)
logical_or = _binary("logical_or", "Elementwise logical or.", inplace=False)
logical_xor = _binary("logical_xor", "Elementwise logical xor.", inplace=False)
pow = _binary("pow", "Elementwise x1 ** x2.")  # noqa: A001
floor_divide = _binary("floor_divide", "Elementwise floor division.")
remainder = _binary("remainder", "Elementwise modulus with the sign of the divisor.")
atan2 = _binary("atan2", "Elementwise arctangent of x1/x2 choosing the quadrant.", inplace=False)
hypot = _binary("hypot", "Elementwise hypotenuse.", inplace=False)
copysign = _binary("copysign", "Elementwise copysign.", inplace=False)
bitwise_left_shift = _binary("bitwise_left_shift", "Elementwise left shift.")
bitwise_right_shift = _binary("bitwise_right_shift", "Elementwise right shift.")
logaddexp = _binary("logaddexp", "Elementwise log(exp(x1) + exp(x2)).", inplace=False)
nextafter = _binary("nextafter", "Next representable value after x1 towards x2.", inplace=False)

# functions of the reference's ufunc extension module (dpnp/backend/extensions/ufunc), which the
# dpnp layer wraps the same way as the tensor functions above
fabs = _unary("fabs", "Elementwise absolute value of a floating array.")
degrees = _unary("degrees", "Radians to degrees.")
radians = _unary("radians", "Degrees to radians.")
sinc = _unary("sinc", "Normalised sinc, sin(pi x) / (pi x).")
spacing = _unary("spacing", "Distance to the nearest adjacent number.")
bitwise_count = _unary("bitwise_count", "Number of set bits of the absolute value.")
erfc = _unary("erfc", "Complementary error function.")
erfcx = _unary("erfcx", "Scaled complementary error function exp(x**2) erfc(x).")
erfinv = _unary("erfinv", "Inverse of the error function.")
erfcinv = _unary("erfcinv", "Inverse of the complementary error function.")
i0 = _unary("i0", "Modified Bessel function of the first kind, order 0.")
fmax = _binary("fmax", "Elementwise maximum; a NaN operand is ignored.", inplace=False)
fmin = _binary("fmin", "Elementwise minimum; a NaN operand is ignored.", inplace=False)
fmod = _binary("fmod", "Elementwise C remainder (sign of the dividend).", inplace=False)
logaddexp2 = _binary("logaddexp2", "Elementwise log2(2**x1 + 2**x2).", inplace=False)
heaviside = _binary("heaviside", "Heaviside step function; x2 where x1 == 0.", inplace=False)
gcd = _binary("gcd", "Elementwise greatest common divisor.", inplace=False)
lcm = _binary("lcm", "Elementwise lowest common multiple.", inplace=False)
