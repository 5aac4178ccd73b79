"""The host side of the polled pair count (no GPU): `poll_host_word` waits for a kernel's store into a pinned word,
falls back to synchronising the stream when the store does not show up in time, and says which of the three it was."""
import numpy as np

from d3gs_research_amd.render import poll_host_word

PENDING = -3


def _clock(step):
    t = [0.0]

    def now():
        t[0] += step
        return t[0]
    return now


def test_store_arrives_while_polling():
    word = np.array([PENDING], np.int64)
    calls = []
    reads = [0]

    class Word:                       # the word changes under the poller's eyes, as a device store would
        def __getitem__(self, i):
            reads[0] += 1
            if reads[0] == 5:
                word[0] = 1234
            return word[i]
    assert poll_host_word(Word(), PENDING, 1.0, lambda: calls.append("sync"), clock=_clock(0.001)) == "polled"
    assert not calls and word[0] == 1234


def test_falls_back_to_a_stream_synchronisation():
    word = np.array([PENDING], np.int64)

    def sync():                       # the stream runs dry: by then the kernel has stored
        word[0] = 77
    assert poll_host_word(word, PENDING, 0.02, sync, clock=_clock(0.005)) == "synced"
    assert word[0] == 77


def test_reports_a_word_that_never_changes():
    word = np.array([PENDING], np.int64)
    calls = []
    assert poll_host_word(word, PENDING, 0.02, lambda: calls.append(1), clock=_clock(0.005)) == "never"
    assert calls == [1] and word[0] == PENDING


def test_a_status_is_a_value_like_any_other():
    word = np.array([-2], np.int64)       # a give-up status replaces the count: it has arrived
    assert poll_host_word(word, PENDING, 0.02, lambda: None) == "polled"
