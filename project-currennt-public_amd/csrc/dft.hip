// Multi-resolution STFT spectral loss (seven amplitude / spectrum distances) and its gradient for gfx950, with
// an in-house radix-4 FFT.
//
// Reference behaviour: helpers/FFTMat.cu (FrameSignal :282-312, distances :473-628, gradients :760-900,
// cleanDummyGradients :456-471, collectGrad :965-1006, drivers :1246-1274, :1350-1475, :1637-1770,
// :1833-1886) and layers/DFTErrorPostoutputLayer.cu (:1186-1244, :1699-1714, :1782-1885).  The reference
// runs about a dozen launches and three cuFFT calls per resolution and waveform, with every intermediate
// (framed signals, spectra, per-bin differences, framed gradients) in device memory.
//
// Here a frame stays in one workgroup's LDS end to end, all resolutions of a call are one launch, and nothing
// but the waveforms and the gradient touches HBM:
//   frame + window source and target  ->  ONE complex FFT of z = source + i*target in LDS (both real
//   spectra are recovered from Z[b] and Z[N-b])  ->  per-bin distance, loss partial and gradient spectrum,
//   written back as its Hermitian extension  ->  inverse FFT in LDS  ->  windowed overlap-add straight into
//   the per-sample gradient with float atomics.
// A workgroup makes several such passes (short transforms more than long ones, so that the workgroups of all
// resolutions carry similar work), loads its twiddles once, fetches the next pass's samples while it computes,
// and adds its loss partial to the per-waveform sums once at its end.
// The forward transform is decimation-in-frequency (natural order in, bit-reversed out), the per-bin stage
// addresses bins through the bit-reversal, and the inverse is decimation-in-time (bit-reversed in, natural
// out), so no reordering pass exists; two butterfly stages share a barrier as one radix-4 butterfly.  Twiddles
// (one run per stage, so that a stage reads consecutive LDS words) and the window (with the reference's
// constant 3.141215) are tabulated in double on the host.  Transform conventions are cuFFT's: unnormalised,
// N/2+1 bins, the imaginary parts of the DC and Nyquist bins do not enter the inverse.
#include "common.hpp"

#include <cmath>
#include <cstring>
#include <new>
#include <vector>

namespace cnt {
namespace {

constexpr int kMaxRes = 3;
constexpr int kMaxWavesPerLaunch = 32;

struct DftParams {
    // per resolution: log2 of the fft length, frame length, frame shift, blocks along x that carry frames
    int logn[kMaxRes], Nw[kMaxRes], Hs[kMaxRes], nblocks[kMaxRes];
    const float2 *twiddle[kMaxRes];  // N entries, stage by stage: entry 2^s + k = exp(-2*pi*i*k / 2^(s+1)), k < 2^s
    const float *window[kMaxRes];    // Nw entries
    int max_length;      // samples per waveform buffer
    int n_waves, n_res;

    int lengths[kMaxWavesPerLaunch];
    float gamma, log_floor;
    float zeta;          // weight of the cosine phase distance; 0 = not evaluated
    const float *source, *target;
    float *grad;    // n_waves x max_length, accumulated over resolutions
    float *errors;  // n_waves x n_res amplitude distances, followed by n_waves x n_res phase distances if zeta > 0
};

__host__ __device__ inline int frame_count(int length, int Nw, int Hs) {
    return length < Nw ? 1 : 1 + (length - Nw) / Hs;
}

// The reference's floors and constants (helpers/FFTMat.hpp: FFT_KLD_FLOOR_NUM, FFT_IS_FLOOR_NUM,
// FFT_SPEC_LOG_MSE_CONST)
constexpr float kKldFloor = 0.00001f;
constexpr float kIsFloor = 0.00001f;
constexpr float kSpecLogMseConst = 1.0f;

// Distance of one bin and the gradient spectrum of that bin, for source spectrum (sx, sy) and target spectrum
// (tx, ty).  Distance functors: helpers/FFTMat.cu:473-628; gradient functors: :760-900.  DIS is the reference's
// specDisType: 0 log-amplitude MSE, 1 KLD of amplitudes, 2 MSE of squared amplitudes, 3 log of the complex
// spectral distance, 4 complex spectral MSE, 5 amplitude ratio, 6 Itakura-Saito.
template <int DIS>
__device__ inline void bin_distance(float sx, float sy, float tx, float ty, float log_floor, float &e, float &gx,
                                    float &gy) {
    const float s2 = sx * sx + sy * sy, t2 = tx * tx + ty * ty;
    if (DIS == 1) {
        const float s = sqrtf(s2 + kKldFloor), t = sqrtf(t2 + kKldFloor);
        e = t * safe_log(t / s) - t + s;
        const float aux = 1.0f - t / s;
        gx = aux * sx / s;
        gy = aux * sy / s;
    } else if (DIS == 2) {
        const float aux = s2 - t2;
        e = aux * aux;
        gx = aux * sx;
        gy = aux * sy;
    } else if (DIS == 3) {
        const float dx = sx - tx, dy = sy - ty;
        const float aux = dx * dx + dy * dy + kSpecLogMseConst;
        e = safe_log(aux);
        gx = dx / aux;
        gy = dy / aux;
    } else if (DIS == 4) {
        const float dx = sx - tx, dy = sy - ty;
        e = dx * dx + dy * dy;
        gx = dx;
        gy = dy;
    } else if (DIS == 5) {
        const float tf = t2 + kKldFloor;
        const float aux = (s2 + kKldFloor) / tf - 1.0f;
        e = aux * aux;
        gx = aux * sx / tf;
        gy = aux * sy / tf;
    } else if (DIS == 6) {
        const float sf = s2 + kIsFloor;
        const float aux = sqrtf(t2 + kIsFloor) / sqrtf(sf);
        e = aux - safe_log(aux) - 1.0f;
        gx = sx / sf * (1.0f - aux);
        gy = sy / sf * (1.0f - aux);
    } else {
        const float spec = s2 + log_floor;
        const float d = safe_log(spec) - safe_log(t2 + log_floor);
        e = d * d;
        gx = d * sx / spec;
        gy = d * sy / spec;
    }
}

// Cosine phase distance 1 - cos(arg S - arg T) of one bin and its gradient spectrum (helpers/FFTMat.cu:630-656
// phaseDistance, :862-878 PhaseGrad; FFT_AMP_MIN_NUM floors the amplitude product, FFT_KLD_FLOOR_NUM the
// gradient's denominator).
constexpr float kAmpMin = 0.0000001f;
__device__ inline void bin_phase(float sx, float sy, float tx, float ty, float &e, float &gx, float &gy) {
    float amp = sqrtf(sx * sx + sy * sy) * sqrtf(tx * tx + ty * ty);
    if (amp < kAmpMin) {
        e = 0.0f;
        amp = kAmpMin;
    } else {
        e = 1.0f - (sx * tx + sy * ty) / amp;
    }
    const float spec = sx * sx + sy * sy + kKldFloor;
    const float fac = (sy * tx - sx * ty) / amp;
    gx = -fac * sy / spec;
    gy = fac * sx / spec;
}

constexpr int kMaxLogN = 12;

// One block = passes of FPB frames of resolution `res` of one waveform.  lds: max(1024, N) + N complex words.
template <int LOGN, int DIS>
__device__ __forceinline__ void dft_frames(const DftParams &p, const int res, float2 *__restrict__ lds,
                                           float (*err_part)[4]) {
    constexpr int N = 1 << LOGN;
    float2 *__restrict__ zbuf = lds;                      // frame storage: FPB * N = max(1024, N) complex words
    float2 *__restrict__ tw = lds + (N > 1024 ? N : 1024);  // N twiddles
    constexpr int HALF = N / 2;
    constexpr int QUARTER = N / 4;
    constexpr int TPF = QUARTER < 256 ? QUARTER : 256;  // threads per frame: one per radix-4 butterfly up to N = 1024
    constexpr int FPB = 256 / TPF;                      // frames per block
    static_assert(FPB * N <= (N > 1024 ? N : 1024), "frame storage: max(1024, N) complex words");

    constexpr int EPT = N / TPF;  // samples per thread and frame

    const int tid = threadIdx.x;
    const int fl = tid / TPF, ft = tid % TPF;  // frame slot in the block, thread within the frame
    float2 *zf = zbuf + fl * N;                // this frame's storage
    const int Nw = p.Nw[res], Hs = p.Hs[res];
    const float *__restrict__ win = p.window[res];
    const int wave_id = blockIdx.y;
    const int length = p.lengths[wave_id];
    const int Kvalid = frame_count(length, Nw, Hs);
    const int kstep = p.nblocks[res] * FPB;  // frames between two passes of this block
    const float *src = p.source + (size_t)wave_id * p.max_length;
    const float *tgt = p.target + (size_t)wave_id * p.max_length;
    float *g = p.grad + (size_t)wave_id * p.max_length;
    const bool phase = p.zeta > 0.0f;
    const float inv = 1.0f / (float)((HALF + 1) * Kvalid);
    const float scale = phase ? inv : p.gamma * inv;
    float err = 0.0f, err_ph = 0.0f;

    // windowed samples of frame k, source in x and target in y; zero outside the window, the waveform and Kvalid
    auto fetch = [&](const int k, float2 (&v)[EPT]) {
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const int j = ft + e * TPF, pos = k * Hs + j;
            v[e] = make_float2(0.0f, 0.0f);
            if (k < Kvalid && j < Nw && pos < length) {
                const float w = win[j];
                v[e] = make_float2(src[pos] * w, tgt[pos] * w);
            }
        }
    };

    int k0 = blockIdx.x * FPB;  // first frame of the pass; the same for every thread, so the barriers are uniform
    if (k0 >= Kvalid) return;
    for (int i = tid; i < N; i += 256) tw[i] = p.twiddle[res][i];
    float2 cur[EPT];
    fetch(k0 + fl, cur);
    for (; k0 < Kvalid; k0 += kstep) {
        const int k = k0 + fl;
        const bool active = k < Kvalid;
#pragma unroll
        for (int e = 0; e < EPT; ++e) zf[ft + e * TPF] = cur[e];
        __syncthreads();
        // the next pass's samples travel while this pass computes
        if (k0 + kstep < Kvalid) fetch(k + kstep, cur);

        // forward: decimation in frequency, two stages (s, s - 1) per barrier as one radix-4 butterfly on the words
        // base + {0, q, 2q, 3q}, q = 2^(s-1); the twiddle of the second pair of stage s is -i times the first's
#pragma unroll 1
        for (int s = LOGN - 1; s >= 1; s -= 2) {
            const int q = 1 << (s - 1);
            for (int i = ft; i < QUARTER; i += TPF) {
                const int j = i & (q - 1);
                const int base = ((i >> (s - 1)) << (s + 1)) + j;
                const float2 x0 = zf[base], x1 = zf[base + q], x2 = zf[base + 2 * q], x3 = zf[base + 3 * q];
                const float2 w1 = tw[2 * q + j], w2 = tw[q + j];
                const float2 y0 = make_float2(x0.x + x2.x, x0.y + x2.y), d02 = make_float2(x0.x - x2.x, x0.y - x2.y);
                const float2 y1 = make_float2(x1.x + x3.x, x1.y + x3.y), d13 = make_float2(x1.y - x3.y, x3.x - x1.x);
                const float2 y2 = make_float2(d02.x * w1.x - d02.y * w1.y, d02.x * w1.y + d02.y * w1.x);
                const float2 y3 = make_float2(d13.x * w1.x - d13.y * w1.y, d13.x * w1.y + d13.y * w1.x);
                const float2 e01 = make_float2(y0.x - y1.x, y0.y - y1.y), e23 = make_float2(y2.x - y3.x, y2.y - y3.y);
                zf[base] = make_float2(y0.x + y1.x, y0.y + y1.y);
                zf[base + q] = make_float2(e01.x * w2.x - e01.y * w2.y, e01.x * w2.y + e01.y * w2.x);
                zf[base + 2 * q] = make_float2(y2.x + y3.x, y2.y + y3.y);
                zf[base + 3 * q] = make_float2(e23.x * w2.x - e23.y * w2.y, e23.x * w2.y + e23.y * w2.x);
            }
            __syncthreads();
        }
        if (LOGN & 1) {  // the last stage on its own: neighbours, twiddle 1
            for (int i = ft; i < HALF; i += TPF) {
                const float2 u = zf[2 * i], v = zf[2 * i + 1];
                zf[2 * i] = make_float2(u.x + v.x, u.y + v.y);
                zf[2 * i + 1] = make_float2(u.x - v.x, u.y - v.y);
            }
            __syncthreads();
        }

        // per-bin stage on the pairs (b, N-b); bin b lives at position bitrev(b)
        // With the phase term both gradient spectra are weighted here and share the inverse transform (the
        // reference runs a second framing / FFT / inverse FFT / overlap-add for it,
        // layers/DFTErrorPostoutputLayer.cu:1246-1295).
        // Stored position q holds bin bitrev(q).  Thread index t walks the even positions 2t (bins below N/2) and
        // pairs each with the position of bin N - b, which for a wave's consecutive t are consecutive words too;
        // walking the bins in natural order instead puts a wave's reads into two LDS banks.  Bins 0 (position 0)
        // and N/2 (position 1) pair with themselves.
        auto bin = [&](const int pb, const int pnb) {
            const float2 zb = zf[pb], zn = zf[pnb];
            // S = (Z[b] + conj(Z[N-b])) / 2,  T = (Z[b] - conj(Z[N-b])) / (2i)
            const float sx = 0.5f * (zb.x + zn.x), sy = 0.5f * (zb.y - zn.y);
            const float tx = 0.5f * (zb.y + zn.y), ty = -0.5f * (zb.x - zn.x);
            float e, gx, gy;
            bin_distance<DIS>(sx, sy, tx, ty, p.log_floor, e, gx, gy);
            if (active) err += e;
            if (phase) {
                float pe, px, py;
                bin_phase(sx, sy, tx, ty, pe, px, py);
                if (active) err_ph += pe;
                gx = p.gamma * gx + p.zeta * px;
                gy = p.gamma * gy + p.zeta * py;
            }
            if (pb == pnb) {
                zf[pb] = make_float2(gx, 0.0f);
            } else {
                zf[pb] = make_float2(gx, gy);
                zf[pnb] = make_float2(gx, -gy);
            }
        };
        for (int t = ft; t < HALF; t += TPF) {
            const int b = (int)(__brev((unsigned)(2 * t)) >> (32 - LOGN));
            const int pnb = (int)(__brev((unsigned)((N - b) & (N - 1))) >> (32 - LOGN));
            bin(2 * t, pnb);
        }
        if (ft == 0) bin(1, 1);
        __syncthreads();

        // inverse: decimation in time with conjugated twiddles, unnormalised; stages (s - 1, s) per barrier
        if (LOGN & 1) {
            for (int i = ft; i < HALF; i += TPF) {
                const float2 u = zf[2 * i], v = zf[2 * i + 1];
                zf[2 * i] = make_float2(u.x + v.x, u.y + v.y);
                zf[2 * i + 1] = make_float2(u.x - v.x, u.y - v.y);
            }
            __syncthreads();
        }
#pragma unroll 1
        for (int s = 1 + (LOGN & 1); s < LOGN; s += 2) {
            const int q = 1 << (s - 1);
            for (int i = ft; i < QUARTER; i += TPF) {
                const int j = i & (q - 1);
                const int base = ((i >> (s - 1)) << (s + 1)) + j;
                const float2 x0 = zf[base], x1 = zf[base + q], x2 = zf[base + 2 * q], x3 = zf[base + 3 * q];
                const float2 w1 = tw[2 * q + j], w2 = tw[q + j];
                const float2 v1 = make_float2(x1.x * w2.x + x1.y * w2.y, x1.y * w2.x - x1.x * w2.y);
                const float2 v3 = make_float2(x3.x * w2.x + x3.y * w2.y, x3.y * w2.x - x3.x * w2.y);
                const float2 y0 = make_float2(x0.x + v1.x, x0.y + v1.y), y1 = make_float2(x0.x - v1.x, x0.y - v1.y);
                const float2 y2 = make_float2(x2.x + v3.x, x2.y + v3.y), y3 = make_float2(x2.x - v3.x, x2.y - v3.y);
                const float2 u2 = make_float2(y2.x * w1.x + y2.y * w1.y, y2.y * w1.x - y2.x * w1.y);
                const float2 t3 = make_float2(y3.x * w1.x + y3.y * w1.y, y3.y * w1.x - y3.x * w1.y);
                const float2 u3 = make_float2(-t3.y, t3.x);  // conj(-i * w1) = i * conj(w1)
                zf[base] = make_float2(y0.x + u2.x, y0.y + u2.y);
                zf[base + q] = make_float2(y1.x + u3.x, y1.y + u3.y);
                zf[base + 2 * q] = make_float2(y0.x - u2.x, y0.y - u2.y);
                zf[base + 3 * q] = make_float2(y1.x - u3.x, y1.y - u3.y);
            }
            __syncthreads();
        }

        // windowed overlap-add; frames at or beyond Kvalid contribute nothing
        if (active) {
            for (int j = ft; j < Nw; j += TPF) {
                const int pos = k * Hs + j;
                if (pos < length) atomicAdd(&g[pos], scale * zf[j].x * win[j]);
            }
        }
        __syncthreads();  // the next pass overwrites the frame storage
    }

    for (int o = 32; o > 0; o >>= 1) {
        err += __shfl_xor(err, o);
        err_ph += __shfl_xor(err_ph, o);
    }
    if ((tid & 63) == 0) {
        err_part[0][tid >> 6] = err;
        err_part[1][tid >> 6] = err_ph;
    }
    __syncthreads();
    if (tid < 2 && (tid == 0 || phase)) {
        const float e = (err_part[tid][0] + err_part[tid][1] + err_part[tid][2] + err_part[tid][3]) * inv;
        if (e != 0.0f) atomicAdd(&p.errors[tid * p.n_waves * p.n_res + wave_id * p.n_res + res], e);
    }
}

// All resolutions of a call in one launch: blockIdx.z selects the resolution, blockIdx.x the group of frames
// (blocks beyond a resolution's last frame leave at once), blockIdx.y the waveform.
template <int DIS>
__global__ __launch_bounds__(256) void dft_loss_kernel(const DftParams p) {
    // sized by the launch for the call's longest transform; every instantiation places its tables at fixed offsets
    extern __shared__ __attribute__((aligned(16))) float2 dft_lds[];
    __shared__ float err_part[2][4];
    const int res = blockIdx.z;
    if ((int)blockIdx.x >= p.nblocks[res]) return;
    switch (p.logn[res]) {
        case 5: dft_frames<5, DIS>(p, res, dft_lds, err_part); break;
        case 6: dft_frames<6, DIS>(p, res, dft_lds, err_part); break;
        case 7: dft_frames<7, DIS>(p, res, dft_lds, err_part); break;
        case 8: dft_frames<8, DIS>(p, res, dft_lds, err_part); break;
        case 9: dft_frames<9, DIS>(p, res, dft_lds, err_part); break;
        case 10: dft_frames<10, DIS>(p, res, dft_lds, err_part); break;
        case 11: dft_frames<11, DIS>(p, res, dft_lds, err_part); break;
        default: dft_frames<12, DIS>(p, res, dft_lds, err_part); break;
    }
}

__global__ void dft_backward_kernel(int max_length, int n_waves, DftParams p, float *__restrict__ prev_errors) {
    const size_t count = (size_t)max_length * n_waves;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const int w = (int)(i / max_length), t = (int)(i % max_length);
        prev_errors[i] = t < p.lengths[w] ? p.grad[i] : 0.0f;
    }
}

typedef void (*dft_kernel_t)(const DftParams);
dft_kernel_t pick_dft_kernel(int dis_type) {
    switch (dis_type) {
        case 0: return dft_loss_kernel<0>;
        case 1: return dft_loss_kernel<1>;
        case 2: return dft_loss_kernel<2>;
        case 3: return dft_loss_kernel<3>;
        case 4: return dft_loss_kernel<4>;
        case 5: return dft_loss_kernel<5>;
        case 6: return dft_loss_kernel<6>;
        default: return nullptr;
    }
}

}  // namespace
}  // namespace cnt

struct cnt_dft {
    cnt_dft_desc desc;
    int logn[cnt::kMaxRes];
    float2 *twiddle[cnt::kMaxRes];
    float *window[cnt::kMaxRes];
    float *grad;  // max_waves x max_length
    int lengths[cnt::kMaxWavesPerLaunch];
    int n_waves;  // of the last forward
};

extern "C" {

int cnt_dft_destroy(cnt_dft *h) {
    if (!h) return CNT_OK;
    for (int r = 0; r < cnt::kMaxRes; ++r) {
        if (h->twiddle[r]) (void)hipFree(h->twiddle[r]);
        if (h->window[r]) (void)hipFree(h->window[r]);
    }
    if (h->grad) (void)hipFree(h->grad);
    delete h;
    return CNT_OK;
}

int cnt_dft_create(const cnt_dft_desc *desc, cnt_dft **out) {
    using namespace cnt;
    CNT_REQUIRE(desc && out, "dft_create: null argument");
    CNT_REQUIRE(desc->n_res >= 1 && desc->n_res <= kMaxRes, "dft_create: %d resolutions, supported 1..%d", desc->n_res,
                kMaxRes);
    CNT_REQUIRE(desc->max_length > 0 && desc->max_waves >= 1 && desc->max_waves <= kMaxWavesPerLaunch,
                "dft_create: max_length must be positive and max_waves in 1..%d", kMaxWavesPerLaunch);
    // the reference implements the Hann window (default) and the square window, and the amplitude / spectrum
    // distances 0..6; its phase distances are a separate driver and are not built
    CNT_REQUIRE(desc->spec_dis_type >= 0 && desc->spec_dis_type <= 6, "dft_create: specDisType %d outside 0..6",
                desc->spec_dis_type);
    CNT_REQUIRE(desc->zeta >= 0.0f, "dft_create: negative zeta");
    CNT_REQUIRE(desc->zeta == 0.0f || desc->phase_dis_type == 0,
                "dft_create: phaseDisType %d; only 0 (cosine distance) is built", desc->phase_dis_type);
    cnt_dft *h = new (std::nothrow) cnt_dft();
    CNT_REQUIRE(h != nullptr, "dft_create: out of host memory");
    std::memset(h, 0, sizeof(*h));
    h->desc = *desc;
    hipError_t err = hipSuccess;
    for (int r = 0; r < desc->n_res && err == hipSuccess; ++r) {
        const int N = desc->fft_length[r], Nw = desc->frame_length[r], Hs = desc->frame_shift[r];
        int logn = 0;
        while ((1 << logn) < N) ++logn;
        if ((1 << logn) != N || logn < 5 || logn > kMaxLogN || Nw < 2 || Nw > N || Hs < 1) {
            set_error("dft_create: resolution %d has fftLength %d, frameLength %d, frameShift %d; supported: fftLength a "
                      "power of two in 32..4096, 2 <= frameLength <= fftLength, frameShift >= 1", r, N, Nw, Hs);
            cnt_dft_destroy(h);
            return CNT_ERR_ARG;
        }
        h->logn[r] = logn;
        // one run of twiddles per butterfly stage, so that a stage reads consecutive LDS words
        std::vector<float2> tw((size_t)N, make_float2(1.0f, 0.0f));
        for (int half = 1; half < N; half *= 2)
            for (int k2 = 0; k2 < half; ++k2) {
                const double a = -3.14159265358979323846 * k2 / half;
                tw[(size_t)(half + k2)] = make_float2((float)std::cos(a), (float)std::sin(a));
            }
        std::vector<float> win((size_t)Nw);
        for (int j = 0; j < Nw; ++j)
            win[(size_t)j] = desc->window_type[r] == 1 ? 1.0f
                                                       : (float)(0.5 * (1 - std::cos(2.0 * 3.141215 * j / (Nw - 1))));
        err = hipMalloc(reinterpret_cast<void **>(&h->twiddle[r]), tw.size() * sizeof(float2));
        if (err == hipSuccess) err = hipMemcpy(h->twiddle[r], tw.data(), tw.size() * sizeof(float2), hipMemcpyHostToDevice);
        if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->window[r]), win.size() * sizeof(float));
        if (err == hipSuccess) err = hipMemcpy(h->window[r], win.data(), win.size() * sizeof(float), hipMemcpyHostToDevice);
    }
    if (err == hipSuccess)
        err = hipMalloc(reinterpret_cast<void **>(&h->grad), (size_t)desc->max_waves * desc->max_length * sizeof(float));
    // a 4096-point transform takes 64 KB of LDS for its frame and twiddles, beyond what a launch may ask for unannounced
    for (int r = 0; r < desc->n_res && err == hipSuccess; ++r)
        if (desc->fft_length[r] > 2048)
            err = hipFuncSetAttribute(reinterpret_cast<const void *>(pick_dft_kernel(desc->spec_dis_type)),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 4096 * (int)sizeof(float2));
    if (err != hipSuccess) {
        set_error("dft_create: %s", hipGetErrorString(err));
        cnt_dft_destroy(h);
        return CNT_ERR_HIP;
    }
    *out = h;
    return CNT_OK;
}

static void fill_params(const cnt_dft *h, cnt::DftParams &p) {
    std::memset(&p, 0, sizeof(p));
    p.max_length = h->desc.max_length;
    p.n_waves = h->n_waves;
    p.n_res = h->desc.n_res;
    for (int w = 0; w < h->n_waves; ++w) p.lengths[w] = h->lengths[w];
    p.gamma = h->desc.gamma;
    p.log_floor = h->desc.log_floor;
    p.zeta = h->desc.zeta;
    p.grad = h->grad;
    for (int r = 0; r < h->desc.n_res; ++r) {
        p.logn[r] = h->logn[r];
        p.Nw[r] = h->desc.frame_length[r];
        p.Hs[r] = h->desc.frame_shift[r];
        p.twiddle[r] = h->twiddle[r];
        p.window[r] = h->window[r];
    }
}

int cnt_dft_forward(cnt_dft *h, void *stream_, int n_waves, const int *lengths, const float *source,
                    const float *target, float *errors_dev) {
    using namespace cnt;
    CNT_REQUIRE(h && lengths && source && target && errors_dev, "dft_forward: null argument");
    CNT_REQUIRE(n_waves >= 1 && n_waves <= h->desc.max_waves, "dft_forward: %d waveforms, handle allows 1..%d", n_waves,
                h->desc.max_waves);
    for (int w = 0; w < n_waves; ++w)
        CNT_REQUIRE(lengths[w] >= 1 && lengths[w] <= h->desc.max_length, "dft_forward: length %d of waveform %d outside 1..%d",
                    lengths[w], w, h->desc.max_length);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    h->n_waves = n_waves;
    for (int w = 0; w < n_waves; ++w) h->lengths[w] = lengths[w];
    CNT_TRY(fill_zero_pair(stream, h->grad, (size_t)n_waves * h->desc.max_length, errors_dev,
                           (size_t)n_waves * h->desc.n_res * (h->desc.zeta > 0.0f ? 2 : 1)));
    int max_len = 0;
    for (int w = 0; w < n_waves; ++w) max_len = lengths[w] > max_len ? lengths[w] : max_len;
    DftParams p;
    fill_params(h, p);
    p.source = source; p.target = target; p.errors = errors_dev;
    // A block of a short transform makes several passes over its waveform's frames, so that the blocks of all
    // resolutions carry about the work of one pass of the longest transform (work per pass: N * log2 N per frame,
    // 256 / (N/4) frames per pass below N = 1024).
    const long max_passes = 8;
    int gx = 1;
    long work_max = 1;
    size_t lds_bytes = 0;
    for (int r = 0; r < h->desc.n_res; ++r) {
        const long n = h->desc.fft_length[r];
        const long w = (n < 1024 ? 1024 : n) * p.logn[r];
        work_max = w > work_max ? w : work_max;
        const size_t b = (size_t)((n < 1024 ? 1024 : n) + n) * sizeof(float2);
        lds_bytes = b > lds_bytes ? b : lds_bytes;
    }
    for (int r = 0; r < h->desc.n_res; ++r) {
        const long n = h->desc.fft_length[r];
        const int quarter = (int)(n / 4);
        const int fpb = quarter < 256 ? 256 / quarter : 1;
        const int kmax = frame_count(max_len, p.Nw[r], p.Hs[r]);
        long passes = work_max / ((n < 1024 ? 1024 : n) * p.logn[r]);
        passes = passes < 1 ? 1 : passes > max_passes ? max_passes : passes;
        const int groups = (kmax + fpb - 1) / fpb;
        p.nblocks[r] = (int)((groups + passes - 1) / passes);
        gx = p.nblocks[r] > gx ? p.nblocks[r] : gx;
    }
    {
        ProfileScope prof(stream, "dft_loss");
        hipLaunchKernelGGL(pick_dft_kernel(h->desc.spec_dis_type), dim3(gx, n_waves, h->desc.n_res), dim3(256), lds_bytes, stream,
                           p);
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}

int cnt_dft_backward(cnt_dft *h, void *stream_, float *prev_errors) {
    using namespace cnt;
    CNT_REQUIRE(h && prev_errors, "dft_backward: null argument");
    CNT_REQUIRE(h->n_waves > 0, "dft_backward: forward has not been called");
    DftParams p;
    fill_params(h, p);
    const size_t count = (size_t)h->desc.max_length * h->n_waves;
    size_t blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    ProfileScope prof(static_cast<hipStream_t>(stream_), "dft_backward");
    hipLaunchKernelGGL(dft_backward_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream_),
                       h->desc.max_length, h->n_waves, p, prev_errors);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

}  // extern "C"
