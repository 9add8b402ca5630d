"""Rotations and their Wigner-D matrices, for the equivariance identities of the test-suite.

Counterparts of the reference's test helpers SO3element (SO3/SO3element.hpp:45-57: a random orthonormal 3x3 matrix
with positive determinant) and SO3irrep.matrix (SO3/SO3irrep.hpp:38-103: z-y-z Euler angles read off the matrix,
D[m1,m2] = d^l_{m2,m1}(beta) e^{i m1 alpha} e^{i m2 gamma})."""
import math

import torch


class SO3element(torch.Tensor):

    @classmethod
    def identity(cls):
        return SO3element(torch.eye(3))

    @classmethod
    def random(cls):
        q, r = torch.linalg.qr(torch.randn(3, 3, dtype=torch.float64))
        q = q * torch.sign(torch.diagonal(r))
        if torch.det(q) < 0:
            q = -q
        return SO3element(q.to(torch.float32))

    def inv(self):
        return SO3element(self.t())


def _littled(l, m1, m2, beta):
    """Wigner small-d element in the summation the reference uses (SO3/SO3irrep.hpp:66-103)."""
    x = 0.0
    c, s = math.cos(beta / 2), math.sin(beta / 2)
    for k in range(max(0, m1 - m2), min(l + m1, l - m2) + 1):
        a = (math.lgamma(l + m1 + 1) + math.lgamma(l - m1 + 1) + math.lgamma(l + m2 + 1) + math.lgamma(l - m2 + 1)) / 2
        a -= math.lgamma(l + m1 - k + 1) + math.lgamma(k + 1) + math.lgamma(m2 - m1 + k + 1) + math.lgamma(l - m2 - k + 1)
        sign = 1 - 2 * ((m2 - m1 + k) % 2)
        x += sign * c ** (2 * l + m1 - m2 - 2 * k) * s ** (m2 - m1 + 2 * k) * math.exp(a)
    return x


class SO3irrep:

    def __init__(self, l):
        assert l >= 0
        self.l = l

    def matrix(self, R):
        R = torch.as_tensor(R, dtype=torch.float64)
        r22 = float(R[2, 2])
        beta = math.acos(max(-1.0, min(1.0, r22)))
        if abs(r22) < 1 - 1e-6:
            alpha = math.atan2(float(R[0, 2]), -float(R[1, 2]))
            gamma = math.atan2(float(R[2, 0]), float(R[2, 1]))
        elif r22 >= 1 - 1e-6:
            alpha, gamma = math.atan2(float(R[1, 0]), float(R[0, 0])), 0.0
        else:
            alpha, gamma = math.atan2(-float(R[1, 0]), -float(R[0, 0])), 0.0
        return self.matrix_euler(alpha, beta, gamma)

    def matrix_euler(self, alpha, beta, gamma):
        l = self.l
        M = torch.zeros(2 * l + 1, 2 * l + 1, dtype=torch.complex128)
        for m1 in range(-l, l + 1):
            for m2 in range(-l, l + 1):
                d = _littled(l, m2, m1, beta)
                M[m1 + l, m2 + l] = d * complex(math.cos(m1 * alpha), math.sin(m1 * alpha)) * \
                    complex(math.cos(m2 * gamma), math.sin(m2 * gamma))
        return M.to(torch.complex64)
