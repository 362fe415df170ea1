// Which layers the Winograd kernels take: their buffer offsets are 32-bit, and two of them keep the top bits of an offset
// for "outside the tensor" marks. One definition for the launchers (which refuse) and the host layer's planner (which
// then keeps the layer on the implicit-GEMM kernels). No HIP types here.
#pragma once

namespace alpha {

// Which of the two layouts of the transformed filter a layer uses (a function of the reduced channel count alone: the
// transform does not know the rest of the layer): grouped U[16][IC/4][OC][4] for the persistent kernel, else U[16][IC][OC].
inline bool winograd_grouped_filter(int IC) { return IC >= 16 && IC % 16 == 0; }

// F(2x2,3x3) in forward form: R channels reduced, P produced, input N x IH x IW x R, output N x OH x OW x P.
// Backward-data is the same with (OH, OW, OC) as the input side and (IH, IW, IC) as the output side.
inline bool winograd_forward_fits(int N, int IH, int IW, int R, int OH, int OW, int P)
{
    if (N < 1 || R < 1 || P < 1 || IH < 1 || IW < 1 || OH < 1 || OW < 1) return false;
    const long in_bytes = 4L * N * IH * IW * R, out_bytes = 4L * N * OH * OW * P, u_bytes = 64L * R * P;
    const long tiles = (long)N * ((OH + 1) / 2) * ((OW + 1) / 2);
    if (in_bytes >= (1L << 31) || u_bytes >= (1L << 31) || tiles >= (1L << 30)) return false;
    if (winograd_grouped_filter(R)) {   // the persistent kernel: output offsets carry a 2 GB "outside" mark; items of 32 tiles x 64 channels
        if (out_bytes > (1L << 30)) return false;
        if (((tiles + 31) / 32) * ((P + 63) / 64) >= (1L << 30)) return false;
    }
    return true;
}

// F(3x3,2x2) backward-filter: patch offsets are a row term plus a column term that mark "outside" by 2 GB and 1 GB, so X
// (and one pixel beyond it) must end below 1 GB.
inline bool winograd_deltaW_fits(int N, int IH, int IW, int IC, int OH, int OW, int OC)
{
    if (N < 1 || IH < 1 || IW < 1 || OH < 1 || OW < 1 || IC < 4 || OC < 4 || (OC & 3)) return false;
    const long x_bytes = 4L * N * IH * IW * IC, y_bytes = 4L * N * OH * OW * OC;
    const long tiles = (long)N * ((OH + 1) / 2) * ((OW + 1) / 2);
    return x_bytes + 8L * IC <= (1L << 30) && y_bytes < (1L << 31) && tiles < (1L << 30);
}

}  // namespace alpha
