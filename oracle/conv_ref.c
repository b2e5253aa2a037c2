/* Brute-force restatement of the Connect6 policy/value forward pass in plain C.
 *
 * TEST INFRASTRUCTURE ONLY: the shipped library never links or loads this.
 * It exists to pin the PyTorch restatement (oracle/torch_ref.py) without going
 * through any library convolution: every output is a literal triple loop over
 * (input channel, ky, kx) in double precision.
 *
 * Follows, in the reference repository:
 *   connect6/model.py:52-66    same-padded stride-1 convolutions with bias
 *   connect6/model.py:67,106   SiLU after every convolution
 *   connect6/model.py:70,108   1x1 policy conv, row-major flatten a = r*n + c
 *   connect6/model.py:74-75,109-110   1x1 value conv -> mean over board -> tanh
 *
 * Layouts are PyTorch's: x [B,Cin,n,n], conv weight [Cout,Cin,k,k], all fp32.
 * Weights of all layers are passed concatenated in layer order, biases likewise.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

static double silu(double v) { return v / (1.0 + exp(-v)); }

/* one same-padded conv + bias (+ SiLU) on a single board, double precision */
static void conv_board(const double *in, int cin, int n, const float *w, const float *b,
                       int cout, int k, int act, double *out)
{
    int pad = k / 2;
    for (int o = 0; o < cout; ++o)
        for (int r = 0; r < n; ++r)
            for (int c = 0; c < n; ++c) {
                double acc = b ? (double)b[o] : 0.0;
                for (int i = 0; i < cin; ++i)
                    for (int ky = 0; ky < k; ++ky) {
                        int rr = r + ky - pad;
                        if (rr < 0 || rr >= n) continue;
                        for (int kx = 0; kx < k; ++kx) {
                            int cc = c + kx - pad;
                            if (cc < 0 || cc >= n) continue;
                            acc += (double)w[((o * cin + i) * k + ky) * k + kx] *
                                   in[(i * n + rr) * n + cc];
                        }
                    }
                out[(o * n + r) * n + c] = act ? silu(acc) : acc;
            }
}

/* returns 0 on success */
int c6ref_forward(const float *x, long batch, int n, int in_channels, int layers,
                  const int *kernels, const int *channels, const float *conv_w,
                  const float *conv_b, const float *pol_w, const float *pol_b,
                  const float *val_w, const float *val_b, float *logits, float *value)
{
    int cmax = in_channels;
    for (int l = 0; l < layers; ++l)
        if (channels[l] > cmax) cmax = channels[l];
    size_t plane = (size_t)n * n;
    double *a = (double *)malloc(sizeof(double) * cmax * plane);
    double *c = (double *)malloc(sizeof(double) * cmax * plane);
    double *pm = (double *)malloc(sizeof(double) * plane);
    if (!a || !c || !pm) return 1;
    for (long bi = 0; bi < batch; ++bi) {
        for (size_t j = 0; j < in_channels * plane; ++j) a[j] = x[bi * in_channels * plane + j];
        const float *w = conv_w, *b = conv_b;
        int cin = in_channels;
        for (int l = 0; l < layers; ++l) {
            conv_board(a, cin, n, w, b, channels[l], kernels[l], 1, c);
            w += (size_t)channels[l] * cin * kernels[l] * kernels[l];
            b += channels[l];
            cin = channels[l];
            double *t = a; a = c; c = t;
        }
        conv_board(a, cin, n, pol_w, pol_b, 1, 1, 0, pm);
        if (logits)
            for (size_t j = 0; j < plane; ++j) logits[bi * plane + j] = (float)pm[j];
        conv_board(a, cin, n, val_w, val_b, 1, 1, 0, pm);
        double s = 0.0;
        for (size_t j = 0; j < plane; ++j) s += pm[j];
        if (value) value[bi] = (float)tanh(s / (double)plane);
    }
    free(a); free(c); free(pm);
    return 0;
}
