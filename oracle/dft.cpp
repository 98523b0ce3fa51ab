// CPU oracle, DFT (STFT spectral) loss -- TEST INFRASTRUCTURE ONLY (see oracle_common.h).
//
// Restates /root/reference/CURRENNT_codes/currennt_lib/src:
//   helpers/FFTMat.cu:282-312      FrameSignal: Hann window with the constant 3.141215, zero padding to the
//                                  FFT length, evaluated in double and rounded once
//   helpers/FFTMat.cu:473-496      log-amplitude distance per bin, d = safeLog(|S|^2+f) - safeLog(|T|^2+f)
//   helpers/FFTMat.cu:760-782      gradient per bin, G = d * S / (|S|^2 + f)
//   helpers/FFTMat.cu:498-628      the other amplitude / spectrum distances (specDisType 1..6), :784-900 their
//                                  gradients; constants helpers/FFTMat.hpp (FFT_KLD_FLOOR_NUM, FFT_IS_FLOOR_NUM,
//                                  FFT_SPEC_LOG_MSE_CONST); double literals in the reference promote the
//                                  expression they stand in to double, restated as such
//   helpers/FFTMat.cu:630-656      phaseDistance (cosine distance), :862-878 PhaseGrad, drivers :1500-1636,
//                                  :1775-1830; layers/DFTErrorPostoutputLayer.cu:1246-1295 (own framing, FFT,
//                                  inverse FFT and collectGrad(zeta) for the phase term)
//   helpers/FFTMat.cu:456-471      cleanDummyGradients
//   helpers/FFTMat.cu:965-1006     collectGrad (windowed overlap-add, scale gamma / (bins * validFrames))
//   helpers/FFTMat.cu:1137-1147    frame / bin counts;  :1152-1202 zero fill beyond the signal length
//   helpers/FFTMat.cu:1350-1475, 1637-1770, 1833-1886   drivers
//   layers/DFTErrorPostoutputLayer.cu:1186-1244, 1699-1714, 1849-1885
// The reference calls cuFFT for the transforms (helpers/FFTMat.cu:1324-1348) and has no host FFT.  The
// transforms here follow cuFFT's published conventions: R2C is the unnormalised forward DFT with
// exp(-i*theta), keeping N/2+1 bins; C2R is the unnormalised inverse of the Hermitian extension and ignores
// the imaginary parts of the DC and Nyquist bins.  They are computed in double (radix-2) and rounded to
// float, i.e. this is the mathematical DFT; parity unpinned at the cuFFT boundary itself (no cuFFT output
// exists in the reference to compare with), pinned against numpy.fft and a brute-force DFT in the tests.
#include "currennt_oracle.h"
#include "oracle_common.h"

#include <cmath>
#include <complex>
#include <vector>

namespace {

typedef std::complex<double> cd;
constexpr double kPiExact = 3.14159265358979323846;
constexpr double kPiWindow = 3.141215;  // the reference's constant inside the window

void fft_pow2(std::vector<cd> &a, bool inverse) {
    const size_t n = a.size();
    for (size_t i = 1, j = 0; i < n; ++i) {
        size_t bit = n >> 1;
        for (; j & bit; bit >>= 1) j ^= bit;
        j ^= bit;
        if (i < j) std::swap(a[i], a[j]);
    }
    for (size_t len = 2; len <= n; len <<= 1) {
        const double ang = 2.0 * kPiExact / (double)len * (inverse ? 1.0 : -1.0);
        for (size_t i = 0; i < n; i += len)
            for (size_t k = 0; k < len / 2; ++k) {
                const cd w(std::cos(ang * (double)k), std::sin(ang * (double)k));
                const cd u = a[i + k], v = a[i + k + len / 2] * w;
                a[i + k] = u + v;
                a[i + k + len / 2] = u - v;
            }
    }
}

int frame_count(int signal_length, int frame_length, int frame_shift) {
    if (signal_length < frame_length) return 1;
    return 1 + (signal_length - frame_length) / frame_shift;
}

float window_product(float raw, int pos, int frame_length, int window_type) {
    if (window_type == 1) return raw;  // square window
    return (float)(raw * 0.5 * (1 - std::cos(2.0 * kPiWindow * pos / (frame_length - 1))));
}

// helpers/FFTMat.hpp
constexpr double kKldFloor = 0.00001, kIsFloor = 0.00001, kSpecLogMseConst = 1.0, kAmpMin = 0.0000001;
constexpr int kPhaseCos = 100;  // internal selector of the cosine phase distance

// first pass of specAmpDistance (helpers/FFTMat.cu:1350-1475): x = distance, y = value kept for the gradient
void bin_distance(int dis_type, float log_floor, float sx, float sy, float tx, float ty, float &x, float &y) {
    switch (dis_type) {
        case 1: {  // SpecAmpDistance_AMP_KLD
            const float s = (float)std::sqrt(sx * sx + sy * sy + kKldFloor);
            const float t = (float)std::sqrt(tx * tx + ty * ty + kKldFloor);
            x = t * orc::safe_log(t / s) - t + s;
            y = (float)(1.0 - t / s);
            break;
        }
        case 2:  // SpecAmpDistance_AMP_MSE
            y = (sx * sx + sy * sy) - (tx * tx + ty * ty);
            x = y * y;
            break;
        case 3:  // SpecAmpDistance_SPEC_LOG_MSE
            y = (float)((sx - tx) * (sx - tx) + (sy - ty) * (sy - ty) + kSpecLogMseConst);
            x = orc::safe_log(y);
            break;
        case 4:  // SpecAmpDistance_SPEC_MSE
            y = 0.0f;
            x = (sx - tx) * (sx - tx) + (sy - ty) * (sy - ty);
            break;
        case 5:  // SpecAmpDistance_AMP_RATIO
            y = (float)((sx * sx + sy * sy + kKldFloor) / (tx * tx + ty * ty + kKldFloor) - 1.0);
            x = y * y;
            break;
        case kPhaseCos: {  // phaseDistance
            y = (float)(std::sqrt(sx * sx + sy * sy) * std::sqrt(tx * tx + ty * ty));
            if (y < kAmpMin) {
                x = 0.0f;
                y = (float)kAmpMin;
            } else {
                x = (float)(1.0 - (sx * tx + sy * ty) / y);
            }
            break;
        }
        case 6: {  // SpecAmpDistance_AMP_IS
            const float sa = (float)std::sqrt(sx * sx + sy * sy + kIsFloor);
            const float ta = (float)std::sqrt(tx * tx + ty * ty + kIsFloor);
            y = ta / sa;
            x = (float)(y - orc::safe_log(y) - 1.0);
            break;
        }
        default: {  // SpecAmpDistance_AMP_LOG_MSE
            const float d = orc::safe_log(sx * sx + sy * sy + log_floor) - orc::safe_log(tx * tx + ty * ty + log_floor);
            y = d;
            x = d * d;
        }
    }
}

// second pass (helpers/FFTMat.cu:1637-1770): (x, y) <- gradient spectrum, y on entry is what pass one left
void bin_gradient(int dis_type, float log_floor, float sx, float sy, float tx, float ty, float &x, float &y) {
    const float keep = y;
    switch (dis_type) {
        case 1: {  // SpecAmpDistance_AMP_KLD_Grad
            const float spec = (float)std::sqrt(sx * sx + sy * sy + kKldFloor);
            x = keep * sx / spec;
            y = keep * sy / spec;
            break;
        }
        case 2:  // SpecAmpDistance_AMP_MSE_Grad
            x = keep * sx;
            y = keep * sy;
            break;
        case 3:  // SpecAmpDistance_SPEC_LOG_MSE_Grad
            x = (sx - tx) / keep;
            y = (sy - ty) / keep;
            break;
        case 4:  // SpecAmpDistance_SPEC_MSE_Grad
            x = sx - tx;
            y = sy - ty;
            break;
        case 5: {  // SpecAmpDistance_AMP_RATIO_Grad
            const float spec = (float)(tx * tx + ty * ty + kKldFloor);
            x = keep * sx / spec;
            y = keep * sy / spec;
            break;
        }
        case kPhaseCos: {  // PhaseGrad
            const float spec = (float)(sx * sx + sy * sy + kKldFloor);
            const float fac = (sy * tx - sx * ty) / keep;
            x = (float)(fac * (-1.0) * sy / spec);
            y = fac * sx / spec;
            break;
        }
        case 6: {  // SpecAmpDistance_AMP_IS_Grad
            const float spec = (float)(sx * sx + sy * sy + kIsFloor);
            x = (float)(sx / spec * (1.0 - keep));
            y = (float)(sy / spec * (1.0 - keep));
            break;
        }
        default: {  // SpecAmpDistance_AMP_LOG_MSE_Grad
            const float spec = sx * sx + sy * sy + log_floor;
            x = keep * sx / spec;
            y = keep * sy / spec;
        }
    }
}

}  // namespace

extern "C" {

int orc_dft_frame_count(int signal_length, int frame_length, int frame_shift) {
    return frame_count(signal_length, frame_length, frame_shift);
}

// out holds n/2+1 interleaved (re, im) pairs
void orc_dft_r2c(int n, const float *in, float *out) {
    std::vector<cd> a((size_t)n);
    for (int i = 0; i < n; ++i) a[(size_t)i] = cd(in[i], 0.0);
    fft_pow2(a, false);
    for (int b = 0; b <= n / 2; ++b) {
        out[2 * b] = (float)a[(size_t)b].real();
        out[2 * b + 1] = (float)a[(size_t)b].imag();
    }
}

void orc_dft_c2r(int n, const float *in, float *out) {
    std::vector<cd> a((size_t)n);
    a[0] = cd(in[0], 0.0);
    a[(size_t)n / 2] = cd(in[2 * (n / 2)], 0.0);
    for (int b = 1; b < n / 2; ++b) {
        a[(size_t)b] = cd(in[2 * b], in[2 * b + 1]);
        a[(size_t)(n - b)] = std::conj(a[(size_t)b]);
    }
    fft_pow2(a, true);
    for (int i = 0; i < n; ++i) out[i] = (float)a[(size_t)i].real();
}

// One resolution, one waveform.  source/target hold max_length samples (content beyond `length` is taken
// as zero, as the reference's buffers are cleared there).  grad receives max_length values.
float orc_dft_spectral_loss(int dis_type, int fft_length, int frame_length, int frame_shift, int window_type,
                            int max_length, int length, float gamma, float log_floor, const float *source,
                            const float *target, float *grad) {
    const int N = fft_length, B = N / 2 + 1;
    const int Kmax = frame_count(max_length, frame_length, frame_shift);
    const int Kvalid = frame_count(length, frame_length, frame_shift);
    std::vector<float> src((size_t)max_length, 0.0f), tgt((size_t)max_length, 0.0f);
    for (int i = 0; i < length; ++i) {
        src[(size_t)i] = source[i];
        tgt[(size_t)i] = target[i];
    }
    std::vector<float> fs((size_t)Kmax * N), ft((size_t)Kmax * N), fg((size_t)Kmax * N);
    for (int k = 0; k < Kmax; ++k)
        for (int j = 0; j < N; ++j) {
            const bool in = j < frame_length;
            // the last frames of the buffer may reach past max_length only when max_length < frame_length
            const int pos = k * frame_shift + j;
            const float rs = (in && pos < max_length) ? src[(size_t)pos] : 0.0f;
            const float rt = (in && pos < max_length) ? tgt[(size_t)pos] : 0.0f;
            fs[(size_t)k * N + j] = in ? window_product(rs, j, frame_length, window_type) : 0.0f;
            ft[(size_t)k * N + j] = in ? window_product(rt, j, frame_length, window_type) : 0.0f;
        }
    std::vector<float> S((size_t)Kmax * B * 2), T((size_t)Kmax * B * 2), Dm((size_t)Kmax * B * 2);
    for (int k = 0; k < Kmax; ++k) {
        orc_dft_r2c(N, &fs[(size_t)k * N], &S[(size_t)k * B * 2]);
        orc_dft_r2c(N, &ft[(size_t)k * N], &T[(size_t)k * B * 2]);
    }
    for (size_t i = 0; i < (size_t)Kmax * B; ++i)
        bin_distance(dis_type, log_floor, S[2 * i], S[2 * i + 1], T[2 * i], T[2 * i + 1], Dm[2 * i], Dm[2 * i + 1]);
    const float factor = (float)(B * Kvalid);
    float err = 0.0f;
    for (size_t i = 0; i < (size_t)B * Kvalid; ++i) err += Dm[2 * i] / factor;
    for (size_t i = 0; i < (size_t)Kmax * B; ++i)
        bin_gradient(dis_type, log_floor, S[2 * i], S[2 * i + 1], T[2 * i], T[2 * i + 1], Dm[2 * i], Dm[2 * i + 1]);
    for (int k = 0; k < Kmax; ++k) orc_dft_c2r(N, &Dm[(size_t)k * B * 2], &fg[(size_t)k * N]);
    for (int k = 0; k < Kmax; ++k)
        for (int j = 0; j < N; ++j)
            if (j > frame_length || k >= Kvalid) fg[(size_t)k * N + j] = 0.0f;
    const float scale = gamma / (float)(B * Kvalid);
    for (int t = 0; t < max_length; ++t) {
        const int k0 = (t >= frame_length) ? (1 + (t - frame_length) / frame_shift) : 0;
        int k1 = t / frame_shift + 1;
        k1 = k1 < Kmax ? k1 : Kmax;
        float acc = 0.0f;
        for (int k = k0; k < k1; ++k) {
            const int pos = t - k * frame_shift;
            const float g = fg[(size_t)k * N + pos];
            if (window_type == 1) acc += g;
            else acc = (float)((double)acc + g * 0.5 * (1 - std::cos(2.0 * kPiWindow * pos / (frame_length - 1))));
        }
        grad[t] = acc * scale;
    }
    return err;
}

// the phase term of one resolution: distance and gradient scaled by zeta
float orc_dft_phase_loss(int fft_length, int frame_length, int frame_shift, int window_type, int max_length,
                         int length, float zeta, const float *source, const float *target, float *grad) {
    return orc_dft_spectral_loss(kPhaseCos, fft_length, frame_length, frame_shift, window_type, max_length, length,
                                 zeta, 0.0f, source, target, grad);
}

float orc_dft_logamp_loss(int fft_length, int frame_length, int frame_shift, int window_type, int max_length,
                          int length, float gamma, float log_floor, const float *source, const float *target,
                          float *grad) {
    return orc_dft_spectral_loss(0, fft_length, frame_length, frame_shift, window_type, max_length, length, gamma,
                                 log_floor, source, target, grad);
}

}  // extern "C"
