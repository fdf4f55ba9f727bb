// Written by tab_amd/tuning/fit_conv_shape_model.py from tab_amd/tuning/conv_shape_training_timings.txt: do not edit.
// Fitted 2026-11-25 on the kernels of commit d089cb0 (and the working tree on top of it).
// Cost model of the matrix-core workgroup shapes: predicted duration (us) = kConvShapeCost[type][i] . f for the shape
// kConvShapeIds[i], f = {G*n, G*rounds, rounds, n, Y, Y*busy, busy, 1, Y*[G <= 9]} (n = tiles on the busiest CU,
// rounds = refills of that CU, Y = megabytes of output, busy = share of the CUs with work; shape 10, the mixed launch:
// {G*whole, G*quarters, quarters, whole, Y, Y, 1, 1, Y*[G <= 9]}, whole tiles per CU and quarter tiles after them).  Non-negative least squares:
// every feature and every coefficient is >= 0, so a prediction is positive and monotone for any geometry.  Regret of the
// choice against the best measured shape over the 280 fitted cases: 1.29%; with each layer set held out of
// the fit in turn: 1.86%.
#pragma once

namespace tab {

constexpr int kConvShapes = 10, kConvShapeFeatures = 9;
// the shape ids tab_set_conv_kernel(TAB_CONV_MATRIX, id) takes, in the order of the tables below
constexpr int kConvShapeIds[kConvShapes] = {0, 1, 2, 3, 4, 5, 6, 8, 9, 10};
// rows x filters of the workgroup tile and workgroups a CU holds (compiled occupancy), per shape
constexpr int kConvShapeTile[kConvShapes][3] = {{128, 128, 4}, {128, 64, 6}, {64, 64, 8}, {32, 32, 4}, {256, 64, 4}, {256, 128, 2}, {128, 256, 2}, {64, 64, 4}, {128, 128, 2}, {128, 128, 4}};
constexpr float kConvShapeCost[4][kConvShapes][kConvShapeFeatures] = {
    {
        {0.09622f, 0.0755577f, 0.0f, 0.0f, 0.0606748f, 0.0f, 1.7507f, 3.14281f, 0.0612442f},
        {0.0671462f, 0.0682265f, 0.0f, 0.0f, 0.0f, 0.0534564f, 1.63501f, 2.45946f, 0.0502946f},
        {0.0451608f, 0.0317093f, 0.0f, 0.42626f, 0.0f, 0.0f, 0.784499f, 2.03594f, 0.0142967f},
        {0.0269856f, 0.0f, 0.0716856f, 0.263235f, 0.0f, 0.0f, 2.58355f, 0.0f, 0.0f},
        {0.100423f, 0.10475f, 0.0f, 0.0f, 0.0485751f, 0.0f, 2.34609f, 3.21895f, 0.0618952f},
        {0.150327f, 0.110511f, 0.0f, 0.0f, 0.0932148f, 0.0f, 1.78975f, 4.71658f, 0.0422527f},
        {0.128618f, 0.118425f, 0.0f, 0.0f, 0.0723173f, 0.0463867f, 0.743713f, 4.19554f, 0.0173782f},
        {0.0251956f, 0.0396773f, 0.0f, 0.670934f, 0.0254314f, 0.0f, 0.734947f, 3.29611f, 0.0f},
        {0.0628066f, 0.0892484f, 0.826519f, 0.0390676f, 0.112093f, 0.0f, 0.0317503f, 4.3067f, 0.0159801f},
        {0.131062f, 0.0280487f, 1.21232f, 0.0f, 0.0760424f, 0.0f, 2.93196f, 0.0f, 0.0f},
    },
    {
        {0.0865426f, 0.0693587f, 0.0f, 0.0f, 0.0579624f, 0.0f, 1.82022f, 2.9411f, 0.0648396f},
        {0.0586298f, 0.0641694f, 0.0f, 0.209004f, 0.0f, 0.0279674f, 1.52226f, 2.17486f, 0.0554612f},
        {0.0383737f, 0.0306837f, 0.0f, 0.412396f, 0.0f, 0.0f, 0.885265f, 1.92272f, 0.0116986f},
        {0.0210085f, 0.00123058f, 0.326048f, 0.171836f, 0.0f, 0.0f, 2.45928f, 0.0f, 0.0f},
        {0.0943118f, 0.0969396f, 0.0f, 0.0f, 0.0546803f, 0.0f, 2.36483f, 2.9726f, 0.0584947f},
        {0.13924f, 0.0996686f, 0.0f, 0.0f, 0.0861756f, 0.0f, 2.11001f, 4.45851f, 0.0409859f},
        {0.121266f, 0.0798943f, 0.0f, 0.0f, 0.0885932f, 0.0317639f, 0.564441f, 3.91746f, 0.0156865f},
        {0.022049f, 0.0348356f, 0.0f, 0.768156f, 0.0f, 0.0f, 0.620039f, 3.04518f, 0.0f},
        {0.0613883f, 0.0738368f, 1.12291f, 0.0f, 0.0950171f, 0.0f, 0.305162f, 3.77746f, 0.0184637f},
        {0.111417f, 0.0296573f, 0.654945f, 0.0f, 0.0718793f, 0.0f, 3.698f, 0.0f, 0.0f},
    },
    {
        {0.0921608f, 0.0695768f, 0.0f, 0.0f, 0.0494465f, 0.0f, 1.69354f, 3.09981f, 0.0724312f},
        {0.0669284f, 0.0552975f, 0.0f, 0.0f, 0.0f, 0.0334096f, 1.58694f, 2.38494f, 0.0745116f},
        {0.0416222f, 0.0198294f, 0.0f, 0.322649f, 0.0f, 0.0f, 0.74886f, 2.16381f, 0.0347851f},
        {0.0201173f, 0.00501934f, 0.423686f, 0.190298f, 0.0f, 0.0f, 2.50451f, 0.0f, 0.0f},
        {0.101425f, 0.0651953f, 0.174489f, 0.0f, 0.0228169f, 0.0f, 2.59556f, 2.74479f, 0.0876685f},
        {0.152702f, 0.0380489f, 0.0f, 0.0f, 0.083621f, 0.0f, 1.93433f, 4.31916f, 0.0504919f},
        {0.138187f, 0.0742667f, 0.0f, 0.0f, 0.0964049f, 0.0304895f, 0.290869f, 4.27502f, 0.00752971f},
        {0.0234524f, 0.0278454f, 0.0f, 0.699996f, 0.0246471f, 0.0f, 0.61602f, 3.03661f, 0.00496521f},
        {0.0751333f, 0.0522657f, 0.737833f, 0.0181711f, 0.116729f, 0.0f, 0.0f, 4.44661f, 0.00639848f},
        {0.110379f, 0.0315015f, 0.678581f, 0.0f, 0.0755007f, 0.0f, 3.64185f, 0.0f, 0.0f},
    },
    {
        {0.070951f, 0.0583979f, 0.0f, 0.0f, 0.07163f, 0.0f, 1.72993f, 2.88768f, 0.0573304f},
        {0.051832f, 0.0574573f, 0.0f, 0.186692f, 0.0f, 0.00781961f, 1.67776f, 1.99304f, 0.082882f},
        {0.0334607f, 0.0209968f, 0.0f, 0.27473f, 0.0f, 0.0f, 0.746789f, 2.1151f, 0.0449228f},
        {0.0165723f, 0.000672762f, 0.409753f, 0.120531f, 0.0f, 0.0f, 2.55998f, 0.0f, 0.0f},
        {0.0815124f, 0.060848f, 0.0f, 0.0f, 0.0399928f, 0.0f, 2.50892f, 2.79836f, 0.0794404f},
        {0.132555f, 0.0385214f, 0.0f, 0.0f, 0.0873704f, 0.0f, 1.8309f, 4.08767f, 0.049155f},
        {0.123896f, 0.040661f, 0.0f, 0.0f, 0.0945826f, 0.0255268f, 0.42759f, 3.8027f, 0.0161334f},
        {0.0182987f, 0.0251055f, 0.0f, 0.701043f, 0.0083251f, 0.0f, 0.680731f, 2.86485f, 0.00394225f},
        {0.0638827f, 0.0401316f, 1.02065f, 0.0f, 0.103476f, 0.0f, 0.113542f, 3.80058f, 0.0134501f},
        {0.0951952f, 0.0254116f, 0.782349f, 0.0f, 0.0604712f, 0.0f, 3.36749f, 0.0f, 0.0f},
    },
};

}  // namespace tab
