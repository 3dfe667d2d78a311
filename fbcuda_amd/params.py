"""FBFFTParameters: the option/error-code holder of fbfft/FBFFTParameters.h:7-59.

Like the reference's, no transform takes it as an argument (the transforms take
padL / padU directly and never normalise); external callers use it to carry
their choices and to name the ErrorCode values.
"""


class FBFFTParameters:
    # ErrorCode (fbfft/FBFFTParameters.h:9-14); HipError stands where CudaError did
    Success = 0
    UnsupportedSize = 1
    UnsupportedDimension = 2
    HipError = 3
    CudaError = 3

    def __init__(self):
        self._forward = True
        self._normalize = False
        self._pad_left = 0
        self._pad_up = 0

    def forward(self):
        self._forward = True
        return self

    def inverse(self):
        self._forward = False
        return self

    def normalize(self, n):
        self._normalize = bool(n)
        return self

    def withPadLeft(self, p):
        self._pad_left = int(p)
        return self

    def withPadUp(self, p):
        self._pad_up = int(p)
        return self

    def forwardFFT(self):
        return self._forward

    def inverseFFT(self):
        return not self._forward

    def normalizeFFT(self):
        return self._normalize

    def padLeft(self):
        return self._pad_left

    def padUp(self):
        return self._pad_up


def numHermitian(commonCols):
    """Stored bins of a Hermitian half spectrum (fbfft/FBFFTCommon.cuh:19-22)."""
    return commonCols // 2 + 1
