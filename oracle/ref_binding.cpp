// Build glue for oracle/_ref: compiles the reference's CPU codec of the entropy-coded format from where it lies
// (REF_SOURCE, never copied) and exposes its three functions to Python.  The reference declares its Python module in
// its CUDA file, which cannot be compiled here; this file only adds the module declaration.
#include REF_SOURCE

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("embed_rows", &embed_rows);
    m.def("encode", &encode);
    m.def("row_hist", &row_hist);
}
