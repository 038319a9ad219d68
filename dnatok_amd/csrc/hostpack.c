/* dnatok_amd._hostpack: a list of Python strings -> one byte buffer + offsets, in one pass in C.
 *
 * Stands where the reference's binding receives std::vector<std::string> and concatenates it
 * (src/dnatok_bpe_kernel/dnatok_bpe.cu:872-887) and where its table paths join and encode the
 * batch (src/dna_tokenizer.py:2594-2651): the bytes go straight into a caller-owned (pinned)
 * buffer, with no joined string, no bytes object and no Python-level loop over the rows.
 *
 *   pack_strings(seqs, address, capacity, utf8) -> (n, total, longest, bytes_at) or -needed
 *
 * Layout written at `address`: int64 offsets[n + 1], then, at the next multiple of 256 bytes
 * (`bytes_at`), the rows' bytes back to back.  utf8 = 0: one byte per character, characters
 * above U+007F become '?'; utf8 = 1: the UTF-8 encoding.  When `capacity` is too small nothing is
 * written and the negated number of bytes needed is returned.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>
#include <string.h>

static Py_ssize_t row_bytes(PyObject *s, int utf8)
{
    if (PyUnicode_IS_COMPACT_ASCII(s) || !utf8) return PyUnicode_GET_LENGTH(s);
    Py_ssize_t n = 0;
    if (!PyUnicode_AsUTF8AndSize(s, &n)) return -1;      /* cached on the object */
    return n;
}

static PyObject *pack_strings(PyObject *self, PyObject *args)
{
    PyObject *seq;
    unsigned long long address;
    Py_ssize_t capacity;
    int utf8;
    (void)self;
    if (!PyArg_ParseTuple(args, "OKni", &seq, &address, &capacity, &utf8)) return NULL;
    PyObject *fast = PySequence_Fast(seq, "pack_strings: expected a sequence of str");
    if (!fast) return NULL;
    const Py_ssize_t n = PySequence_Fast_GET_SIZE(fast);
    PyObject **items = PySequence_Fast_ITEMS(fast);
    Py_ssize_t total = 0, longest = 0;
    for (Py_ssize_t i = 0; i < n; ++i) {
        if (!PyUnicode_Check(items[i])) {
            Py_DECREF(fast);
            PyErr_SetString(PyExc_TypeError, "pack_strings: every row must be a str");
            return NULL;
        }
        const Py_ssize_t len = row_bytes(items[i], utf8);
        if (len < 0) { Py_DECREF(fast); return NULL; }
        total += len;
        if (len > longest) longest = len;
    }
    const Py_ssize_t bytes_at = ((n + 1) * 8 + 255) & ~(Py_ssize_t)255;
    const Py_ssize_t needed = bytes_at + total;
    if (needed > capacity || address == 0) {
        Py_DECREF(fast);
        return PyLong_FromSsize_t(-needed);
    }
    int64_t *offsets = (int64_t *)(uintptr_t)address;
    uint8_t *out = (uint8_t *)(uintptr_t)address + bytes_at;
    Py_ssize_t at = 0;
    for (Py_ssize_t i = 0; i < n; ++i) {
        PyObject *s = items[i];
        offsets[i] = at;
        const Py_ssize_t chars = PyUnicode_GET_LENGTH(s);
        if (PyUnicode_IS_COMPACT_ASCII(s)) {
            memcpy(out + at, PyUnicode_DATA(s), (size_t)chars);
            at += chars;
        } else if (utf8) {
            Py_ssize_t len = 0;
            const char *p = PyUnicode_AsUTF8AndSize(s, &len);
            if (!p) { Py_DECREF(fast); return NULL; }
            memcpy(out + at, p, (size_t)len);
            at += len;
        } else {
            const int kind = PyUnicode_KIND(s);
            const void *data = PyUnicode_DATA(s);
            for (Py_ssize_t c = 0; c < chars; ++c) {
                const Py_UCS4 ch = PyUnicode_READ(kind, data, c);
                out[at + c] = ch < 128 ? (uint8_t)ch : (uint8_t)'?';
            }
            at += chars;
        }
    }
    offsets[n] = at;
    Py_DECREF(fast);
    return Py_BuildValue("(nnnn)", n, total, longest, bytes_at);
}

static PyMethodDef methods[] = {
    {"pack_strings", pack_strings, METH_VARARGS,
     "pack_strings(seqs, address, capacity, utf8) -> (n, total, longest, bytes_at) or -needed"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_hostpack",
                                    "Strings of a batch into one byte buffer + offsets, in C.", -1, methods,
                                    NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__hostpack(void) { return PyModule_Create(&module); }
