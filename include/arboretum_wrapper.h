/*
 * C-ABI of libarboretum.so: the drop-in boundary.
 *
 * These are the 14 entry points of the reference's python-wrapper
 * (python-wrapper/arboretum_wrapper.h:6-39), with the same names, argument
 * order and meaning, so the reference's ctypes loader
 * (python-package/arboretum/core.py:21-43) binds them unchanged.
 *
 * Convention (python-wrapper/arboretum_wrapper.cu:16-205): every function
 * returns NULL on success or a NUL-terminated message that stays valid until
 * the next failing call on the same thread.  Handles are opaque.  One booster
 * per caller thread; the library is not re-entrant on one handle.
 *
 * Training (AGrowTree) runs on one MI355X through hand-written HIP kernels and
 * fails with an error string when no HIP device is present; the other entry
 * points are host code, as in the reference.
 */
#ifndef ARBORETUM_WRAPPER_H_
#define ARBORETUM_WRAPPER_H_

#ifdef __cplusplus
extern "C" {
#endif

typedef void *VoidPointer;

/* python-wrapper/arboretum_wrapper.cu:16-39.  `data` is row-major
 * [nrow][ncol] fp32 and is copied; `categories` (row-major uint32
 * [nrow][ccol], may be NULL when ccol == 0) is stored but unused by the
 * histogram path, as in the reference; `missing` is accepted and ignored
 * (NaN marks a missing value and always goes right). */
const char *ACreateFromDenseMatrix(const float *data, const unsigned int *categories, int nrow,
                                   int ncol, int ccol, float missing, VoidPointer *out);

/* arboretum_wrapper.cu:41-55: copies nrow floats (regression target / 0-1 label). */
const char *ASetY(VoidPointer data, const float *y);

/* arboretum_wrapper.cu:57-71: copies nrow class ids (multi-class). */
const char *ASetLabel(VoidPointer data, const unsigned char *labels);

/* arboretum_wrapper.cu:73-86: copies nrow sample weights (stored, unused, as
 * in the reference). */
const char *ASetWeights(VoidPointer data, const float *weights);

/* arboretum_wrapper.cu:88-99: parses the JSON configuration
 * (src/core/json_conversion.h:55-167) and creates a booster.  Malformed JSON
 * returns an error string (the reference aborts the process). */
const char *AInitGarden(const char *configuration, VoidPointer *garden);

/* arboretum_wrapper.cu:101-111 -> Garden::GrowTree (src/core/garden.cu:585-625):
 * one boosting round (labels_count trees).  The first call quantises `data`
 * and binds the booster to it.  `grad` must be NULL (the reference ignores a
 * non-NULL gradient, garden.cu:609-614; here it is an error). */
const char *AGrowTree(VoidPointer garden, VoidPointer data, const float *grad);

/* arboretum_wrapper.cu:181-193 -> Garden::UpdateByLastTree (garden.cu:627-635):
 * adds the last round's trees to data->y_hat on the host. */
const char *AAppendLastTree(VoidPointer garden, VoidPointer data);

/* arboretum_wrapper.cu:153-179 -> Garden::GetY (garden.cu:637-641): link
 * function of data->y_hat; *out is released with ADeleteArray. */
const char *AGetY(VoidPointer garden, VoidPointer data, const float **out);

/* arboretum_wrapper.cu:113-139 -> Garden::Predict (garden.cu:643-657):
 * n_rounds == -1 means all; the first min(n_rounds, #trees) trees are used;
 * *out holds nrow * labels_count floats, released with ADeleteArray. */
const char *APredict(VoidPointer garden, VoidPointer data, const float **out, const int n_rounds);

/* arboretum_wrapper.cu:141-145 -> DumpModel (src/core/model_helper.cpp:16-23):
 * JSON {"configuration":..,"model":[..]}; the string belongs to the booster
 * and stays valid until the next ADumpModel or AFreeGarden on it. */
const char *ADumpModel(const char **model, VoidPointer garden);

/* arboretum_wrapper.cu:147-151 -> Garden::Restore (garden.cu:667-677):
 * appends the trees of the "model" array. */
const char *ALoadModel(const char *model, VoidPointer garden);

/* arboretum_wrapper.cu:195-205 */
const char *AFreeDMatrix(VoidPointer ptr);
const char *AFreeGarden(VoidPointer ptr);
const char *ADeleteArray(float *in);

#ifdef __cplusplus
}
#endif
#endif /* ARBORETUM_WRAPPER_H_ */
