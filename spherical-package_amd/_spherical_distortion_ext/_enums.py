"""`_enums`: the interpolation selector shared by every operator.

Values follow ext_modules/include/enums.h:12-16; like the reference's
py::arithmetic enum (include/layers/enum_export.h:10-18) the members convert
to and from integers, and a 0-d integer tensor is accepted by the constructor
(the autograd functions rebuild the enum from a saved tensor).
"""
import enum


class InterpolationType(enum.IntEnum):
    NEAREST = 0
    BILINEAR = 1
    BISPHERICAL = 2

    @classmethod
    def _missing_(cls, value):
        try:
            as_int = int(value)
        except (TypeError, ValueError):
            return None
        for member in cls:
            if member.value == as_int:
                return member
        return None
