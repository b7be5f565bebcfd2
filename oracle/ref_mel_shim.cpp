// Checker infrastructure, not product code: gives tests/golden/make_fixtures.py and the CPU leg of bench.py a
// way to call the reference's log-mel front end directly.  log_mel_spectrogram (src/whisper.cpp:3181-3270) is a
// static function with no public getter for its result, so this translation unit takes the reference's source
// file in from where it lies (-I $(REF)/src, see oracle/Makefile) and adds one exported wrapper behind it.
// Built into oracle/_ref/libref_mel.so; nothing of the reference is copied into this repository.
#include "whisper.cpp"

extern "C" __attribute__((visibility("default")))
int ref_log_mel_spectrogram(const float * samples, int n_samples, const float * filters, int n_mel, int n_threads,
                            float * out, int out_capacity, int * n_len, int * n_len_org) {
    whisper_filters f;
    f.n_mel = n_mel;
    f.n_fft = 1 + WHISPER_N_FFT / 2;
    f.data.assign(filters, filters + (size_t) n_mel * f.n_fft);
    whisper_mel mel;
    whisper_state * st = new whisper_state();
    const bool ok = log_mel_spectrogram(*st, samples, n_samples, WHISPER_SAMPLE_RATE, WHISPER_N_FFT, WHISPER_HOP_LENGTH, n_mel, n_threads, f, false, mel);
    delete st;
    if (!ok) return -1;
    if (n_len) *n_len = mel.n_len;
    if (n_len_org) *n_len_org = mel.n_len_org;
    if (!out) return 0;
    if ((size_t) out_capacity < mel.data.size()) return -2;
    std::copy(mel.data.begin(), mel.data.end(), out);
    return 0;
}
