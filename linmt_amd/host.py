"""ctypes binding of liblinmt_host.so (C facade of the C++ layer classes, include/linmt_host.h).

Python plumbing for the tests and the benchmark only; the computation happens in the C++ classes
and the HIP kernels.  No fallback: a missing library raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblinmt_host.so")
_lib = None


class HostError(RuntimeError):
    pass


class Config(C.Structure):
    _fields_ = [("num_layers", C.c_int), ("lstm_size", C.c_int), ("embedding_size", C.c_int),
                ("source_vocab_size", C.c_int), ("target_vocab_size", C.c_int),
                ("minibatch_size", C.c_int), ("longest_sentence", C.c_int),
                ("attention_mode", C.c_int), ("attention_width", C.c_int), ("feed_input", C.c_int),
                ("sequence_to_sequence", C.c_int), ("clip_cell", C.c_int),
                ("cell_clip_threshold", C.c_float)]


class TrainOptions(C.Structure):
    _fields_ = [("learning_rate", C.c_float), ("grad_clip_mode", C.c_int), ("norm_clip", C.c_float),
                ("individual_clip", C.c_float), ("error_clip_threshold", C.c_float),
                ("dropout_keep", C.c_float), ("dropout_seed", C.c_ulonglong)]


class TuningOptions(C.Structure):
    _fields_ = [("train_file", C.c_char_p), ("dev_file", C.c_char_p),
                ("output_weight_file", C.c_char_p), ("best_model_file", C.c_char_p),
                ("epochs", C.c_int), ("google_learning_rate", C.c_int),
                ("epoch_to_start_halving", C.c_int), ("stanford_learning_rate", C.c_int),
                ("epoch_to_start_halving_full", C.c_int), ("learning_rate_schedule", C.c_int),
                ("decrease_factor", C.c_float), ("margin", C.c_double),
                ("best_model_mode", C.c_int), ("screen_print_rate", C.c_int)]


class TuningEvent(C.Structure):
    _fields_ = [("kind", C.c_int), ("epoch", C.c_int), ("minibatch", C.c_int),
                ("value", C.c_double)]


class DecodingOptions(C.Structure):
    _fields_ = [("model_file", C.c_char_p), ("source_file", C.c_char_p), ("ids_file", C.c_char_p),
                ("final_file", C.c_char_p), ("beam_size", C.c_int), ("penalty", C.c_float),
                ("max_decoding_ratio", C.c_float), ("min_decoding_ratio", C.c_float),
                ("lp_alpha", C.c_float), ("cp_beta", C.c_float), ("diversity", C.c_float),
                ("longest_sentence", C.c_int), ("attention_width", C.c_int),
                ("print_decoding_information", C.c_int),
                ("print_alignments_scores", C.c_int), ("unk_replacement_mode", C.c_int),
                ("sentences_per_batch", C.c_int), ("num_hypotheses", C.c_int),
                ("ensemble_model_files", C.POINTER(C.c_char_p)), ("n_ensemble_models", C.c_int)]


class DecodeOptions(C.Structure):
    _fields_ = [("beam_size", C.c_int), ("max_decoding_ratio", C.c_float),
                ("min_decoding_ratio", C.c_float), ("penalty", C.c_float),
                ("diversity", C.c_float), ("lp_alpha", C.c_float), ("cp_beta", C.c_float),
                ("unk_replacement_mode", C.c_int), ("num_hypotheses", C.c_int)]


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HostError(f"{LIB_PATH} is missing: build it with __graft_entry__.build(); "
                        "there is no CPU fallback")
    # torch brings a HIP runtime of its own: whichever runtime a process loads first has to be the
    # one that initialises the device, so torch goes first wherever both end up in one process
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    lib.lnmt_last_error.restype = C.c_char_p
    lib.lnmt_model_create_scoring.restype = C.c_void_p
    lib.lnmt_model_create_scoring.argtypes = [C.POINTER(Config)]
    lib.lnmt_model_create_decoding.restype = C.c_void_p
    lib.lnmt_model_create_decoding.argtypes = [C.POINTER(Config), C.c_int, C.c_int]
    lib.lnmt_model_create_training.restype = C.c_void_p
    lib.lnmt_model_create_training.argtypes = [C.POINTER(Config), C.POINTER(TrainOptions)]
    lib.lnmt_compute_gradients.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                           C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                           C.c_void_p, C.c_int, C.POINTER(C.c_double)]
    lib.lnmt_compute_gradients_stepwise.argtypes = lib.lnmt_compute_gradients.argtypes
    lib.lnmt_model_get_grad.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_longlong]
    lib.lnmt_update_weights.argtypes = [C.c_void_p, C.POINTER(C.c_double)]
    lib.lnmt_clear_gradients.argtypes = [C.c_void_p]
    lib.lnmt_set_train_modes.argtypes = [C.c_void_p] + [C.c_int] * 6
    lib.lnmt_set_debug_option.argtypes = [C.c_char_p, C.c_int]
    lib.lnmt_set_dropout_seed.argtypes = [C.c_void_p, C.c_ulonglong]
    lib.lnmt_get_dropout_mask.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                          C.c_longlong]
    lib.lnmt_model_destroy.argtypes = [C.c_void_p]
    lib.lnmt_model_destroy.restype = None
    lib.lnmt_model_set_param.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_longlong]
    lib.lnmt_model_get_param.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_longlong]
    lib.lnmt_get_error.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                   C.c_int, C.c_void_p, C.c_int, C.POINTER(C.c_double)]
    lib.lnmt_get_state.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                   C.c_longlong]
    lib.lnmt_decode_batch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                      C.POINTER(DecodeOptions), C.c_void_p, C.c_int, C.c_void_p,
                                      C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.lnmt_decode_batch_ensemble.argtypes = [C.POINTER(C.c_void_p), C.c_int] + \
        lib.lnmt_decode_batch.argtypes[1:]
    lib.lnmt_decode_history.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_int, C.POINTER(C.c_int)]
    lib.lnmt_decode_stream.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                       C.POINTER(DecodeOptions), C.c_void_p, C.c_int, C.c_void_p,
                                       C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.POINTER(C.c_int)]
    lib.lnmt_decode_stream_ensemble.argtypes = [C.POINTER(C.c_void_p), C.c_int] + \
        lib.lnmt_decode_stream.argtypes[1:]
    lib.lnmt_model_stream.restype = C.c_void_p
    lib.lnmt_model_stream.argtypes = [C.c_void_p]
    lib.lnmt_set_split_products.argtypes = [C.c_void_p, C.c_int, C.c_int]
    lib.lnmt_profile_set_level.argtypes = [C.c_void_p, C.c_int]
    lib.lnmt_profile_count.argtypes = [C.c_void_p]
    lib.lnmt_profile_entry.argtypes = [C.c_void_p, C.c_int, C.c_char_p, C.c_int,
                                       C.POINTER(C.c_double), C.POINTER(C.c_double),
                                       C.POINTER(C.c_longlong)]
    lib.lnmt_read_model_information.argtypes = [C.c_char_p, C.POINTER(C.c_int * 9)]
    lib.lnmt_model_load_weights.argtypes = [C.c_void_p, C.c_char_p]
    lib.lnmt_model_dump_model.argtypes = [C.c_void_p, C.c_char_p]
    lib.lnmt_model_file_param.argtypes = [C.c_void_p, C.c_int, C.c_char_p, C.c_int,
                                          C.POINTER(C.c_int), C.POINTER(C.c_int)]
    lib.lnmt_file_helper_create.restype = C.c_void_p
    lib.lnmt_file_helper_create.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, C.c_int]
    lib.lnmt_file_helper_destroy.argtypes = [C.c_void_p]
    lib.lnmt_file_helper_destroy.restype = None
    lib.lnmt_file_helper_read_minibatch.argtypes = [C.c_void_p]
    lib.lnmt_file_helper_get.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_longlong]
    lib.lnmt_file_helper_info.argtypes = [C.c_void_p, C.POINTER(C.c_int * 8)]
    lib.lnmt_decoding.argtypes = [C.POINTER(DecodingOptions), C.POINTER(C.c_int), C.POINTER(C.c_int),
                                  C.POINTER(C.c_longlong), C.POINTER(C.c_longlong),
                                  C.POINTER(C.c_double)]
    lib.lnmt_integerize_file_decoding.argtypes = [C.c_char_p, C.c_char_p, C.c_int, C.c_void_p,
                                                  C.c_longlong, C.c_void_p, C.c_void_p, C.c_int,
                                                  C.POINTER(C.c_int), C.POINTER(C.c_int)]
    lib.lnmt_unint_file.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, C.c_int, C.c_int]
    lib.lnmt_tuning.argtypes = [C.c_void_p, C.POINTER(TuningOptions), C.POINTER(TuningEvent),
                                C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_longlong),
                                C.POINTER(C.c_double), C.POINTER(C.c_float)]
    lib.lnmt_get_perplexity.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_double)]
    lib.lnmt_decoder_sentence_create.restype = C.c_void_p
    lib.lnmt_decoder_sentence_create.argtypes = [C.c_char_p, C.c_int]
    lib.lnmt_decoder_sentence_destroy.restype = None
    lib.lnmt_decoder_sentence_destroy.argtypes = [C.c_void_p]
    lib.lnmt_decoder_sentence_process.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_size_t,
                                                  C.POINTER(C.c_size_t)]
    lib.lnmt_decoder_sentence_unint.argtypes = lib.lnmt_decoder_sentence_process.argtypes
    lib.lnmt_decoder_sentence_integerize.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int,
                                                     C.POINTER(C.c_int)]
    lib.lnmt_decoder_sentence_settings.argtypes = [C.c_void_p, C.POINTER(DecodingOptions),
                                                   C.c_char_p, C.c_size_t]
    lib.python_decoder_init.restype = None
    lib.python_decoder_init.argtypes = [C.c_char_p]
    lib.python_decoder_do_job.restype = C.c_char_p
    lib.python_decoder_do_job.argtypes = [C.c_char_p]
    _lib = lib
    return lib


def _check(rc, what):
    if rc != 0:
        raise HostError(f"{what}: {load().lnmt_last_error().decode('utf-8', 'replace')}")


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class Model:
    def __init__(self, num_layers, lstm_size, source_vocab_size, target_vocab_size,
                 longest_sentence=104, attention_mode=1, attention_width=10, feed_input=True,
                 minibatch_size=1, embedding_size=0, sequence_to_sequence=True, decoding=None,
                 clip_cell=False, cell_clip_threshold=50.0, training=None):
        """decoding=(n_sent, beam) builds the batched decoder; training=dict(learning_rate,
        grad_clip_mode, norm_clip, individual_clip, error_clip_threshold) the training model;
        otherwise the scoring model."""
        self.cfg = Config(num_layers, lstm_size, embedding_size, source_vocab_size,
                          target_vocab_size, minibatch_size, longest_sentence, attention_mode,
                          attention_width, int(feed_input), int(sequence_to_sequence),
                          int(clip_cell), cell_clip_threshold)
        lib = load()
        if decoding is not None:
            self.n_sent, self.beam = decoding
            h = lib.lnmt_model_create_decoding(C.byref(self.cfg), self.n_sent, self.beam)
        elif training is not None:
            t = TrainOptions(training.get("learning_rate", 0.7), training.get("grad_clip_mode", 1),
                             training.get("norm_clip", 5.0), training.get("individual_clip", 0.1),
                             training.get("error_clip_threshold", 1000.0),
                             training.get("dropout_keep", 0.0), training.get("dropout_seed", 1))
            h = lib.lnmt_model_create_training(C.byref(self.cfg), C.byref(t))
        else:
            h = lib.lnmt_model_create_scoring(C.byref(self.cfg))
        if not h:
            raise HostError("model creation failed: "
                            + lib.lnmt_last_error().decode("utf-8", "replace"))
        self.handle = C.c_void_p(h)

    def close(self):
        if getattr(self, "handle", None):
            load().lnmt_model_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def stream(self):
        return load().lnmt_model_stream(self.handle)

    def set_split_products(self, on=True, min_columns=0):
        """Decoding: gate products and output projection from three-way bf16 splits on the bf16
        matrix pipe while at least min_columns hypotheses are alive (lnmt_set_split_products)."""
        _check(load().lnmt_set_split_products(self.handle, int(on), int(min_columns)), "set_split_products")

    def profile(self, level):
        """0 off, 1 output projection only, 2 every launch (HIP events on the model's stream)."""
        _check(load().lnmt_profile_set_level(self.handle, level), "profile_set_level")

    def profile_totals(self):
        """name -> dict(ms, work, launches); matrix products are keyed 'site|kernel instance'."""
        lib = load()
        out = {}
        for i in range(lib.lnmt_profile_count(self.handle)):
            name = C.create_string_buffer(256)
            ms, work, n = C.c_double(0), C.c_double(0), C.c_longlong(0)
            _check(lib.lnmt_profile_entry(self.handle, i, name, 256, C.byref(ms), C.byref(work),
                                          C.byref(n)), "profile_entry")
            out[name.value.decode()] = dict(ms=ms.value, work=work.value, launches=n.value)
        return out

    def set_params(self, params):
        """params: name -> 2-D/1-D array in mathematical layout (rows x cols)."""
        for name, arr in params.items():
            flat = np.ascontiguousarray(np.asarray(arr, np.float32).ravel(order="F"))
            _check(load().lnmt_model_set_param(self.handle, name.encode(), _p(flat), flat.size),
                   f"set_param({name})")

    def get_param(self, name, shape):
        out = np.empty(int(np.prod(shape)), np.float32)
        _check(load().lnmt_model_get_param(self.handle, name.encode(), _p(out), out.size),
               f"get_param({name})")
        return out.reshape(shape, order="F")

    EVENT_KINDS = ("speed", "half_epoch_perplexity", "epoch_perplexity", "learning_rate",
                   "dump_best_model", "epoch_end", "dump_final")

    def tuning(self, train_file, dev_file=None, output_weight_file=None, best_model_file=None,
               epochs=10, google_learning_rate=False, epoch_to_start_halving=6,
               stanford_learning_rate=False, epoch_to_start_halving_full=6,
               learning_rate_schedule=False, decrease_factor=0.5, margin=0.0,
               best_model_mode=False, screen_print_rate=20):
        """Dispatcher::Tuning.  Returns dict(events=[(kind, epoch, minibatch, value)], words,
        seconds, final_learning_rate)."""
        enc = lambda p: None if p is None else os.fsencode(p)  # noqa: E731
        o = TuningOptions(enc(train_file), enc(dev_file), enc(output_weight_file),
                          enc(best_model_file), epochs, int(google_learning_rate),
                          epoch_to_start_halving, int(stanford_learning_rate),
                          epoch_to_start_halving_full, int(learning_rate_schedule),
                          decrease_factor, margin, int(best_model_mode), screen_print_rate)
        cap = 65536
        ev = (TuningEvent * cap)()
        n, words, secs, lr = C.c_int(), C.c_longlong(), C.c_double(), C.c_float()
        _check(load().lnmt_tuning(self.handle, C.byref(o), ev, cap, C.byref(n), C.byref(words),
                                  C.byref(secs), C.byref(lr)), "tuning")
        events = [(self.EVENT_KINDS[ev[i].kind], ev[i].epoch, ev[i].minibatch, ev[i].value)
                  for i in range(min(n.value, cap))]
        return dict(events=events, words=words.value, seconds=secs.value,
                    final_learning_rate=lr.value)

    def get_perplexity(self, path):
        out = C.c_double()
        _check(load().lnmt_get_perplexity(self.handle, os.fsencode(path), C.byref(out)),
               "get_perplexity")
        return out.value

    def load_weights(self, path):
        """NeuralMachineTranslation::LoadWeights: fill the parameters from a reference model file."""
        _check(load().lnmt_model_load_weights(self.handle, os.fsencode(path)), "load_weights")

    def dump_model(self, path):
        """Write a complete reference-format model file (placeholder vocabulary mappings)."""
        _check(load().lnmt_model_dump_model(self.handle, os.fsencode(path)), "dump_model")

    def model_file_order(self):
        """[(name, rows, cols)] in the order the model file stores the matrices."""
        lib, out = load(), []
        name, r, c = C.create_string_buffer(64), C.c_int(), C.c_int()
        n = lib.lnmt_model_file_param(self.handle, 0, name, 64, C.byref(r), C.byref(c))
        if n < 0:
            _check(-1, "model_file_order")
        for i in range(n):
            lib.lnmt_model_file_param(self.handle, i, name, 64, C.byref(r), C.byref(c))
            out.append((name.value.decode(), r.value, c.value))
        return out

    def get_error(self, src, tgt_in, tgt_out, batch_info):
        """src (B,S), tgt_in/tgt_out (B,T) int arrays, -1 padding; returns sum log p(target)."""
        src = np.asfortranarray(src, np.int32) if src is not None else None
        tgt_in = np.asfortranarray(tgt_in, np.int32)
        tgt_out = np.asfortranarray(tgt_out, np.int32)
        B, T = tgt_in.shape
        S = src.shape[1] if src is not None else 0
        bi = None if batch_info is None else np.ascontiguousarray(batch_info, np.int32)
        loss = C.c_double(0)
        _check(load().lnmt_get_error(self.handle, _p(src), S, _p(tgt_in), _p(tgt_out), T, _p(bi), B,
                                     C.byref(loss)), "get_error")
        return loss.value

    def compute_gradients(self, src, tgt_in, tgt_out, batch_info, src_unique, tgt_unique,
                          stepwise=False):
        """Forward + backward of one minibatch (no update); returns sum log p(target).
        stepwise: drive the layers node by node with the reference's calls, in its order."""
        src = np.asfortranarray(src, np.int32) if src is not None else None
        tgt_in = np.asfortranarray(tgt_in, np.int32)
        tgt_out = np.asfortranarray(tgt_out, np.int32)
        B, T = tgt_in.shape
        S = src.shape[1] if src is not None else 0
        bi = None if batch_info is None else np.ascontiguousarray(batch_info, np.int32)
        su = None if src_unique is None else np.ascontiguousarray(src_unique, np.int32)
        tu = np.ascontiguousarray(tgt_unique, np.int32)
        loss = C.c_double(0)
        fn = load().lnmt_compute_gradients_stepwise if stepwise else load().lnmt_compute_gradients
        _check(fn(self.handle, _p(src), S, _p(tgt_in), _p(tgt_out), T,
                  _p(su), 0 if su is None else su.size, _p(tu), tu.size,
                  _p(bi), B, C.byref(loss)), "compute_gradients")
        return loss.value

    def get_grad(self, name, shape):
        out = np.empty(int(np.prod(shape)), np.float32)
        _check(load().lnmt_model_get_grad(self.handle, name.encode(), _p(out), out.size),
               f"get_grad({name})")
        return out.reshape(shape, order="F")

    def update_weights(self):
        """UpdateWeights + ClearGradients; returns the global norm (0 unless grad_clip_mode 2)."""
        nrm = C.c_double(0)
        _check(load().lnmt_update_weights(self.handle, C.byref(nrm)), "update_weights")
        return nrm.value

    def get_dropout_mask(self, kind, side, layer, rows, B, steps):
        """(steps, B, rows) view of the masks of the last compute_gradients call."""
        out = np.empty(rows * B * steps, np.float32)
        _check(load().lnmt_get_dropout_mask(self.handle, kind, side, layer, _p(out), out.size),
               "get_dropout_mask")
        return out.reshape((steps, B, rows))

    def clear_gradients(self):
        _check(load().lnmt_clear_gradients(self.handle), "clear_gradients")

    def set_train_modes(self, source_input_embedding=True, target_input_embedding=True,
                        target_output_embedding=True, source_rnn=True, target_rnn=True,
                        attention_target_rnn=True):
        """The reference's train_*_mode__ switches (finetune = the three embedding groups off)."""
        _check(load().lnmt_set_train_modes(self.handle, int(source_input_embedding),
                                           int(target_input_embedding), int(target_output_embedding),
                                           int(source_rnn), int(target_rnn), int(attention_target_rnn)),
               "set_train_modes")

    def set_dropout_seed(self, seed):
        _check(load().lnmt_set_dropout_seed(self.handle, seed), "set_dropout_seed")

    def decode_history(self, sentence, beam):
        """Beam of sentence `sentence` of the last decode_batch call after every expansion step:
        (tok, backptr, score), each (steps, beam); back-pointers are beam-local."""
        cap = self.cfg.longest_sentence + 2
        tok = np.zeros((cap, beam), np.int32)
        bp = np.zeros((cap, beam), np.int32)
        sc = np.zeros((cap, beam), np.float32)
        n = C.c_int(0)
        _check(load().lnmt_decode_history(self.handle, sentence, _p(tok), _p(bp), _p(sc), cap,
                                          C.byref(n)), "decode_history")
        return tok[:n.value].copy(), bp[:n.value].copy(), sc[:n.value].copy()

    def get_state(self, kind, side, layer, timestep, rows, cols):
        out = np.empty(rows * cols, np.float32)
        _check(load().lnmt_get_state(self.handle, kind, side, layer, timestep, _p(out), out.size),
               "get_state")
        return out.reshape((rows, cols), order="F")

    def decode_batch(self, sentences, beam=12, max_ratio=1.5, min_ratio=0.5, penalty=0.0,
                     diversity=0.0, lp_alpha=0.65, cp_beta=0.20, with_hyps=False, hyp_cap=256,
                     alignments=False, num_hypotheses=1, ensemble=()):
        """alignments=True: the reference's unk_replacement_mode__; results gain best_viterbi.
        num_hypotheses > 1: results gain kbest = [(index into the finished hypotheses, final
        score)], best first.  ensemble: further decoding models whose distributions are averaged
        with this one's before every beam step (EnsembleFactory with several models)."""
        n = len(sentences)
        lengths = np.array([len(s) for s in sentences], np.int32)
        flat = np.ascontiguousarray(np.concatenate([np.asarray(s, np.int32) for s in sentences]))
        cap = self.cfg.longest_sentence + 2
        o = DecodeOptions(beam, max_ratio, min_ratio, penalty, diversity, lp_alpha, cp_beta,
                          int(alignments), int(num_hypotheses))
        kidx = np.full((n, max(1, num_hypotheses)), -1, np.int32)
        kscore = np.zeros((n, max(1, num_hypotheses)), np.float32)
        best = np.zeros((n, cap), np.int32)
        vit = np.full((n, cap), -1, np.int32) if alignments else None
        blen = np.zeros(n, np.int32)
        bscore = np.zeros(n, np.float32)
        steps = np.zeros(n, np.int32)
        nh = np.zeros(n, np.int32)
        ht = hl = hs = None
        if with_hyps:
            ht = np.zeros((n, hyp_cap, cap), np.int32)
            hl = np.zeros((n, hyp_cap), np.int32)
            hs = np.zeros((n, hyp_cap), np.float32)
        handles = (C.c_void_p * (1 + len(ensemble)))(self.handle, *[m.handle for m in ensemble])
        _check(load().lnmt_decode_batch_ensemble(handles, len(handles), _p(flat), _p(lengths), n,
                                                 C.byref(o), _p(best), cap, _p(blen), _p(bscore),
                                                 _p(steps), _p(ht), _p(hl), _p(hs), hyp_cap, _p(nh),
                                                 _p(vit), _p(kidx), _p(kscore)),
               "decode_batch")
        res = []
        for i in range(n):
            r = dict(best=best[i, :blen[i]].copy(), best_score=float(bscore[i]),
                     steps=int(steps[i]), n_hyp=int(nh[i]))
            if with_hyps:
                k = min(int(nh[i]), hyp_cap)
                r["hyps"] = [(ht[i, j, :hl[i, j]].copy(), float(hs[i, j])) for j in range(k)]
            if alignments:
                r["best_viterbi"] = vit[i, :blen[i]].copy()
            r["kbest"] = [(int(a), float(b)) for a, b in zip(kidx[i], kscore[i]) if a >= 0]
            res.append(r)
        return res


def _decode_stream(self, sentences, beam=12, max_ratio=1.5, min_ratio=0.5, penalty=0.0, diversity=0.0,
                   lp_alpha=0.65, cp_beta=0.20, with_hyps=False, hyp_cap=256, alignments=False,
                   num_hypotheses=1, ensemble=()):
    """DecodeStream: any number of sentences through the model's n_sent slots of beam columns, a
    finished sentence's slot going to the next sentence.  Results as decode_batch, in the order of
    `sentences`; self.stream_ticks = steps taken in all."""
    n = len(sentences)
    lengths = np.array([len(s) for s in sentences], np.int32)
    flat = np.ascontiguousarray(np.concatenate([np.asarray(s, np.int32) for s in sentences]))
    cap = self.cfg.longest_sentence + 2
    o = DecodeOptions(beam, max_ratio, min_ratio, penalty, diversity, lp_alpha, cp_beta,
                      int(alignments), int(num_hypotheses))
    kidx = np.full((n, max(1, num_hypotheses)), -1, np.int32)
    kscore = np.zeros((n, max(1, num_hypotheses)), np.float32)
    best = np.zeros((n, cap), np.int32)
    vit = np.full((n, cap), -1, np.int32) if alignments else None
    blen = np.zeros(n, np.int32)
    bscore = np.zeros(n, np.float32)
    steps = np.zeros(n, np.int32)
    nh = np.zeros(n, np.int32)
    ht = hl = hs = None
    if with_hyps:
        ht = np.zeros((n, hyp_cap, cap), np.int32)
        hl = np.zeros((n, hyp_cap), np.int32)
        hs = np.zeros((n, hyp_cap), np.float32)
    ticks = C.c_int(0)
    if ensemble:
        handles = (C.c_void_p * (1 + len(ensemble)))(self.handle, *[m.handle for m in ensemble])
        _check(load().lnmt_decode_stream_ensemble(handles, len(handles), _p(flat), _p(lengths), n,
                                                  C.byref(o), _p(best), cap, _p(blen), _p(bscore),
                                                  _p(steps), _p(ht), _p(hl), _p(hs), hyp_cap, _p(nh),
                                                  _p(vit), _p(kidx), _p(kscore), C.byref(ticks)),
               "decode_stream_ensemble")
    else:
        _check(load().lnmt_decode_stream(self.handle, _p(flat), _p(lengths), n, C.byref(o), _p(best), cap,
                                         _p(blen), _p(bscore), _p(steps), _p(ht), _p(hl), _p(hs), hyp_cap,
                                         _p(nh), _p(vit), _p(kidx), _p(kscore), C.byref(ticks)),
               "decode_stream")
    self.stream_ticks = ticks.value
    res = []
    for i in range(n):
        r = dict(best=best[i, :blen[i]].copy(), best_score=float(bscore[i]), steps=int(steps[i]),
                 n_hyp=int(nh[i]))
        if with_hyps:
            k = min(int(nh[i]), hyp_cap)
            r["hyps"] = [(ht[i, j, :hl[i, j]].copy(), float(hs[i, j])) for j in range(k)]
        if alignments:
            r["best_viterbi"] = vit[i, :blen[i]].copy()
        r["kbest"] = [(int(a), float(b)) for a, b in zip(kidx[i], kscore[i]) if a >= 0]
        res.append(r)
    return res


Model.decode_stream = _decode_stream


def set_debug_option(name, value):
    """lnmt_set_debug_option: a process-wide measurement / test aid of the decode path."""
    _check(load().lnmt_set_debug_option(name.encode(), int(value)), "set_debug_option")


def decoding(model_file, source_file, final_file, ids_file=None, beam=12, penalty=0.0,
             max_ratio=1.5, min_ratio=0.5, lp_alpha=0.65, cp_beta=0.20, diversity=0.0,
             longest_sentence=200, attention_width=10, print_decoding_information=False,
             print_alignments_scores=False, unk_replacement_mode=False, sentences_per_batch=64,
             num_hypotheses=1, ensemble_model_files=()):
    """Dispatcher::Decoding: translate a text file with a reference model file (or with an
    ensemble: model_file plus ensemble_model_files)."""
    enc = lambda p: None if p is None else os.fsencode(p)  # noqa: E731
    more = (C.c_char_p * max(1, len(ensemble_model_files)))(*[enc(f) for f in ensemble_model_files])
    o = DecodingOptions(enc(model_file), enc(source_file), enc(ids_file), enc(final_file), beam,
                        penalty, max_ratio, min_ratio, lp_alpha, cp_beta, diversity,
                        longest_sentence, attention_width, int(print_decoding_information),
                        int(print_alignments_scores), int(unk_replacement_mode),
                        sentences_per_batch, num_hypotheses, more, len(ensemble_model_files))
    n, thrown, sw, tw, secs = C.c_int(), C.c_int(), C.c_longlong(), C.c_longlong(), C.c_double()
    _check(load().lnmt_decoding(C.byref(o), C.byref(n), C.byref(thrown), C.byref(sw), C.byref(tw),
                                C.byref(secs)), "decoding")
    return dict(sentences=n.value, sentences_thrown_away=thrown.value, source_words=sw.value,
                target_words=tw.value, seconds=secs.value)


def integerize_file_decoding(model_file, source_file, max_sent_cutoff):
    """IntegerizeFileDecoding: (list of id arrays in reading order, input line of each, target
    vocabulary size)."""
    lib = load()
    n, v = C.c_int(), C.c_int()
    cap_s, cap_i = 1 << 16, 1 << 22
    ids, lens, lines = np.empty(cap_i, np.int32), np.empty(cap_s, np.int32), np.empty(cap_s, np.int32)
    _check(lib.lnmt_integerize_file_decoding(os.fsencode(model_file), os.fsencode(source_file),
                                             max_sent_cutoff, _p(ids), cap_i, _p(lens), _p(lines),
                                             cap_s, C.byref(n), C.byref(v)),
           "integerize_file_decoding")
    out, at = [], 0
    for i in range(min(n.value, cap_s)):
        out.append(ids[at:at + lens[i]].copy())
        at += lens[i]
    return out, lines[:len(out)].tolist(), v.value


def unint_file(model_file, unint_path, final_path, sequence_to_sequence=True, decoder_mode=True):
    _check(load().lnmt_unint_file(os.fsencode(model_file), os.fsencode(unint_path),
                                  os.fsencode(final_path), int(sequence_to_sequence),
                                  int(decoder_mode)), "unint_file")


class DecoderSentence:
    """The reference's one-sentence decoder (DecoderSentence, src/decoder_sentence.h:22-52):
    configuration file -> model; process(sentence) -> translation text.  load_model=False reads
    the configuration and the vocabularies only (no GPU): integerize / unint / settings work."""

    def __init__(self, config_file, load_model=True):
        self._h = load().lnmt_decoder_sentence_create(os.fsencode(config_file), int(load_model))
        if not self._h:
            raise HostError("DecoderSentence: " + load().lnmt_last_error().decode("utf-8", "replace"))

    def close(self):
        if self._h:
            load().lnmt_decoder_sentence_destroy(self._h)
            self._h = None

    __del__ = close

    def _text(self, fn, sentence, what):
        cap = 1 << 16
        while True:
            buf, need = C.create_string_buffer(cap), C.c_size_t(0)
            rc = fn(self._h, sentence.encode("utf-8"), buf, cap, C.byref(need))
            if rc != 0 and need.value > cap:
                cap = need.value
                continue
            _check(rc, what)
            return buf.value.decode("utf-8", "replace")

    def process(self, sentence):
        return self._text(load().lnmt_decoder_sentence_process, sentence, "DecoderSentence.process")

    def unint(self, sentence):
        return self._text(load().lnmt_decoder_sentence_unint, sentence, "DecoderSentence.unint")

    def integerize(self, sentence):
        """ids in the order the encoder reads them (reversed)."""
        cap = max(16, len(sentence))
        ids, n = np.empty(cap, np.int32), C.c_int(0)
        _check(load().lnmt_decoder_sentence_integerize(self._h, sentence.encode("utf-8"), _p(ids), cap,
                                                       C.byref(n)), "DecoderSentence.integerize")
        return ids[:n.value].copy()

    def settings(self):
        o, name = DecodingOptions(), C.create_string_buffer(4096)
        _check(load().lnmt_decoder_sentence_settings(self._h, C.byref(o), name, 4096),
               "DecoderSentence.settings")
        out = {f: getattr(o, f) for f, _ in DecodingOptions._fields_
               if f not in ("model_file", "source_file", "ids_file", "final_file")}
        out["model_file"] = os.fsdecode(name.value)
        return out


def python_decoder_init(config_file):
    """python_decoder_init of the reference's server library (src/decoder_sentence.cu:847-850)."""
    load().python_decoder_init(os.fsencode(config_file))


def python_decoder_do_job(sentence):
    """python_decoder_do_job (src/decoder_sentence.cu:852-874): bytes in, translation text out."""
    return load().python_decoder_do_job(sentence.encode("utf-8")).decode("utf-8", "replace")


def read_model_information(path):
    """dict of the first line of a reference model file."""
    info = (C.c_int * 9)()
    _check(load().lnmt_read_model_information(os.fsencode(path), C.byref(info)),
           "read_model_information")
    keys = ("num_layers", "lstm_size", "target_vocab_size", "source_vocab_size", "attention_model",
            "feed_input", "multi_source", "combine_lstm", "char_cnn")
    return dict(zip(keys, list(info)))


class FileHelper:
    """The reference's training-file reader (FileHelper, src/file_helper.h): four lines per
    sentence pair; read_minibatch() returns the arrays of one minibatch."""

    ARRAYS = ("source_in", "source_out", "target_in", "target_out", "source_wgrad", "target_wgrad",
              "batch_information")

    def __init__(self, path, minibatch_size, longest_sentence, source_vocab_size,
                 target_vocab_size):
        self.B, self.cap = minibatch_size, minibatch_size * longest_sentence
        self.handle = load().lnmt_file_helper_create(os.fsencode(path), minibatch_size,
                                                     longest_sentence, source_vocab_size,
                                                     target_vocab_size)
        if not self.handle:
            _check(-1, "FileHelper")

    def close(self):
        if self.handle:
            load().lnmt_file_helper_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def read_minibatch(self):
        """(same_epoch, dict): id blocks as (B, length) arrays, the two unique-id lists, the batch
        information and the counters of FileHelper."""
        lib = load()
        rc = lib.lnmt_file_helper_read_minibatch(self.handle)
        if rc < 0:
            _check(-1, "read_minibatch")
        info = (C.c_int * 8)()
        _check(lib.lnmt_file_helper_info(self.handle, C.byref(info)), "file_helper_info")
        S, T = info[0], info[1]
        out = dict(current_source_length=S, current_target_length=T, words_in_minibatch=info[2],
                   nums_lines_in_file=info[5], total_words=info[6], total_target_words=info[7])
        buf = np.empty(max(self.cap, 2 * self.B), np.int32)
        for what, key in enumerate(self.ARRAYS):
            n = lib.lnmt_file_helper_get(self.handle, what, _p(buf), buf.size)
            if n < 0:
                _check(-1, f"file_helper_get({key})")
            a = buf[:n].copy()
            if what < 4:
                a = a.reshape((self.B, S if what < 2 else T), order="F")
            out[key] = a
        return bool(rc), out
