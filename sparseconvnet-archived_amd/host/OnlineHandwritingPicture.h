// Pen strokes as input samples: the reference's OnlineHandwritingPicture
// (OnlineHandwritingPicture.h:8-26), the front-end of its pen-digits, Assamese
// and CASIA online-handwriting drivers, without Armadillo.  A character is a
// list of strokes, a stroke a list of 2-D points; it is fitted into a square
// of side renderSize, every stroke is resampled at constant speed, and the
// samples are binned into the lattice with one of the encodings below.
//
// Not available: the four LogSignature encodings.  They project path
// signatures onto a basis that the reference ships as tables generated with a
// third-party tool (signature.h:1-5, 96-514); those tables are data of the
// reference and are not restated here.  Asking for one of them fails with a
// message.
#pragma once
#include <string>
#include <vector>
#include "Picture.h"

// types.h:29-44 of the reference
enum OnlineHandwritingEncoding {
  Simple,             // 1 feature: samples per cell
  Octogram,           // 8: direction of travel, spread over the two nearest of 8 compass points
  UndirectedOctogram, // 4: the same without orientation
  LogSignature1,
  LogSignature2,
  LogSignature3,
  LogSignature4,
  SpaceTime3d,       // 1 feature, 3-D lattice: the third axis is time (sample number)
  VectorSpaceTime3d  // 3 features, 3-D lattice: count, sum of unit directions
};
extern const int OnlineHandwritingEncodingSize[9];

class OnlineHandwritingPicture : public Picture {
public:
  float penSpeed3d;
  float offset3d;
  std::vector<std::vector<double>> ops; // per stroke: nPoints x 2
  int renderSize;
  OnlineHandwritingEncoding enc;
  OnlineHandwritingPicture(int renderSize, OnlineHandwritingEncoding enc,
                           int label, float penSpeed3d = 0.02f);
  void addStroke(const double *xy, int nPoints);
  // fit centrally in the square [-renderSize/2, renderSize/2]^2
  void normalize();
  Picture *distort(RNG &rng, batchType type);
  void codifyInputData(SparseGrid &grid, std::vector<float> &features,
                       int &nSpatialSites, int spatialSize);
  std::string identify();
};

// points of a stroke at equal arc-length spacing `density` (n = round(length /
// density) * multiplier intervals): OnlineHandwritingPicture.cpp:27-53
std::vector<double> constantSpeed(const std::vector<double> &stroke,
                                  float density, int multiplier = 1);

// The UCI pen-digits files (pendigits-orig.tra / .tes): one picture per
// ".COMMENT <label>" record, strokes between .PEN_DOWN and .PEN_UP, points as
// "x y" with x becoming -column and y the row, each picture normalized
// (SpatiallySparseDatasetPenDigits.cpp:15-63).  Returns the number of pictures
// appended, -1 when the file cannot be opened.
int readPenDigitsFile(std::vector<Picture *> &characters, const char *filename,
                      int renderSize, OnlineHandwritingEncoding enc);
