/* -*- c++ -*- ----------------------------------------------------------
   LAMMPS pair style symmetrix/mace over the MI355X engine (libsymmetrix_amd.so).

   Same commands as the reference pair style (pair_symmetrix/pair_symmetrix_mace.h:16, .cpp:95-153):
       pair_style symmetrix/mace [no_domain_decomposition | mpi_message_passing | no_mpi_message_passing]
       pair_coeff * * model.json El1 El2 ...
   plus the spelling symmetrix/mace/float32 for float32 features with float64 accumulation (the reference has
   that spelling on its Kokkos styles only, pair_symmetrix_mace_kokkos.h:24-26).

   The class holds the LAMMPS-facing part only: neighbour list -> flat edge arrays, LAMMPS communication, scatter
   into atom->f.  Everything between the reference's "begin mace evaluation" and "end mace evaluation" marks lives
   in mace_evaluation.{h,cpp}, which has no LAMMPS types and is built and run by this repository's tests.
------------------------------------------------------------------------- */

#ifdef PAIR_CLASS
// clang-format off
PairStyle(symmetrix/mace,PairSymmetrixMACE);
PairStyle(symmetrix/mace/float32,PairSymmetrixMACEFloat32);
// clang-format on
#else

#ifndef LMP_PAIR_SYMMETRIX_MACE_AMD_H
#define LMP_PAIR_SYMMETRIX_MACE_AMD_H

#include <memory>
#include <string>
#include <vector>

#include "pair.h"

#include "mace_evaluation.h"

namespace LAMMPS_NS {

class PairSymmetrixMACE : public Pair {
 public:
  PairSymmetrixMACE(class LAMMPS *);
  ~PairSymmetrixMACE() override;

  void compute(int, int) override;
  void settings(int, char **) override;
  void coeff(int, char **) override;
  double init_one(int, int) override;
  void init_style() override;
  int pack_forward_comm(int, int *, double *, int, int *) override;
  void unpack_forward_comm(int, int, double *) override;
  int pack_reverse_comm(int, int, double *) override;
  void unpack_reverse_comm(int, int *, double *) override;

 protected:
  enum Mode { NO_DOMAIN_DECOMPOSITION, MPI_MESSAGE_PASSING, NO_MPI_MESSAGE_PASSING };
  Mode mode = NO_DOMAIN_DECOMPOSITION;
  int precision = SMX_FP64;                 // the /float32 style sets SMX_FP32_FEATURES

  std::unique_ptr<MACE> mace;
  std::vector<int> mace_types;              // LAMMPS type - 1 -> species index of the model
  symmetrix_amd::EdgeList edges;            // rebuilt every step from the full neighbour list
  std::vector<double> H1, H1_adj;           // exchange buffers of the mode mpi_message_passing, by atom row
  std::vector<int> node_of_atom;            // atom row -> node (or -1), for the modes that index H1 by node
  std::vector<double> eatom_nodes;

  void allocate();
  void build_edges();                       // local receivers; ghost nodes appended in the mode that wants them
  int width() const { return mace->num_LM * mace->num_channels; }
};

class PairSymmetrixMACEFloat32 : public PairSymmetrixMACE {
 public:
  PairSymmetrixMACEFloat32(class LAMMPS *lmp) : PairSymmetrixMACE(lmp) { precision = SMX_FP32_FEATURES; }
};

}    // namespace LAMMPS_NS

#endif
#endif
