/* ----------------------------------------------------------------------
   LAMMPS pair style symmetrix/mace over the MI355X engine; see pair_symmetrix_mace.h.
   Needs a LAMMPS source tree to compile (this file is the only one here that does).
------------------------------------------------------------------------- */

#include "pair_symmetrix_mace.h"

#include "atom.h"
#include "comm.h"
#include "error.h"
#include "force.h"
#include "memory.h"
#include "neigh_list.h"
#include "neighbor.h"

#include <algorithm>
#include <array>
#include <cmath>
#include <cstring>

using namespace LAMMPS_NS;

namespace {
const std::array<const char *, 118> kSymbols = {
    "H",  "He", "Li", "Be", "B",  "C",  "N",  "O",  "F",  "Ne", "Na", "Mg", "Al", "Si", "P",  "S",  "Cl", "Ar", "K",  "Ca",
    "Sc", "Ti", "V",  "Cr", "Mn", "Fe", "Co", "Ni", "Cu", "Zn", "Ga", "Ge", "As", "Se", "Br", "Kr", "Rb", "Sr", "Y",  "Zr",
    "Nb", "Mo", "Tc", "Ru", "Rh", "Pd", "Ag", "Cd", "In", "Sn", "Sb", "Te", "I",  "Xe", "Cs", "Ba", "La", "Ce", "Pr", "Nd",
    "Pm", "Sm", "Eu", "Gd", "Tb", "Dy", "Ho", "Er", "Tm", "Yb", "Lu", "Hf", "Ta", "W",  "Re", "Os", "Ir", "Pt", "Au", "Hg",
    "Tl", "Pb", "Bi", "Po", "At", "Rn", "Fr", "Ra", "Ac", "Th", "Pa", "U",  "Np", "Pu", "Am", "Cm", "Bk", "Cf", "Es", "Fm",
    "Md", "No", "Lr", "Rf", "Db", "Sg", "Bh", "Hs", "Mt", "Ds", "Rg", "Cn", "Nh", "Fl", "Mc", "Lv", "Ts", "Og"};
}

PairSymmetrixMACE::PairSymmetrixMACE(LAMMPS *lmp) : Pair(lmp)
{
  single_enable = 0;
  restartinfo = 0;
  one_coeff = 1;
  manybody_flag = 1;
  no_virial_fdotr_compute = 1;
  // the message size depends on the model and is set in coeff(); until then a bound that LAMMPS' buffers can hold
  // (zero would break hybrid/overlay, as the reference notes at pair_symmetrix_mace.cpp:42-49)
  comm_forward = 1024;
  comm_reverse = 1024;
}

PairSymmetrixMACE::~PairSymmetrixMACE()
{
  if (allocated) {
    memory->destroy(setflag);
    memory->destroy(cutsq);
  }
}

void PairSymmetrixMACE::allocate()
{
  allocated = 1;
  const int n = atom->ntypes + 1;
  memory->create(setflag, n, n, "pair:setflag");
  memory->create(cutsq, n, n, "pair:cutsq");
  for (int i = 1; i < n; ++i)
    for (int j = i; j < n; ++j) setflag[i][j] = 0;
}

void PairSymmetrixMACE::settings(int narg, char **arg)
{
  if (narg > 1) error->all(FLERR, "Too many pair_style arguments for symmetrix/mace");
  if (narg == 0) {
    mode = comm->nprocs == 1 ? NO_DOMAIN_DECOMPOSITION : MPI_MESSAGE_PASSING;
  } else {
    const std::string m(arg[0]);
    if (m == "no_domain_decomposition") mode = NO_DOMAIN_DECOMPOSITION;
    else if (m == "mpi_message_passing") mode = MPI_MESSAGE_PASSING;
    else if (m == "no_mpi_message_passing") mode = NO_MPI_MESSAGE_PASSING;
    else error->all(FLERR, "The command 'pair_style symmetrix/mace {}' is invalid", m);
  }
  if (mode == NO_DOMAIN_DECOMPOSITION && comm->nprocs != 1)
    error->all(FLERR, "Cannot use no_domain_decomposition with multiple MPI processes");
}

void PairSymmetrixMACE::coeff(int narg, char **arg)
{
  if (!allocated) allocate();
  if (narg != 3 + atom->ntypes) error->all(FLERR, "pair_coeff * * model.json followed by one element per atom type");
  utils::logmesg(lmp, "Loading MACE model from '{}' ({} features) ... ", arg[2],
                 precision == SMX_FP64 ? "float64" : "float32");
  try {
    mace = std::make_unique<MACE>(arg[2], precision);
  } catch (const std::exception &e) {
    error->all(FLERR, "symmetrix/mace: {}", e.what());
  }
  utils::logmesg(lmp, "success\n");

  mace_types.clear();
  for (int a = 3; a < narg; ++a) {
    const auto sym = std::find_if(kSymbols.begin(), kSymbols.end(), [&](const char *s) { return std::strcmp(s, arg[a]) == 0; });
    if (sym == kSymbols.end()) error->all(FLERR, "{} does not appear in the periodic table", arg[a]);
    const int Z = (int) (sym - kSymbols.begin()) + 1;
    const auto it = std::find(mace->atomic_numbers.begin(), mace->atomic_numbers.end(), Z);
    if (it == mace->atomic_numbers.end()) error->all(FLERR, "Problem matching LAMMPS types to MACE types.");
    const int index = (int) (it - mace->atomic_numbers.begin());
    utils::logmesg(lmp, "  mapping LAMMPS type {} ({}) to MACE type {}\n", a - 2, arg[a], index);
    mace_types.push_back(index);
  }
  comm_forward = comm_reverse = mode == MPI_MESSAGE_PASSING ? width() : 0;
  for (int i = 1; i <= atom->ntypes; ++i)
    for (int j = i; j <= atom->ntypes; ++j) setflag[i][j] = 1;
}

double PairSymmetrixMACE::init_one(int i, int j)
{
  if (setflag[i][j] == 0) error->all(FLERR, "All pair coeffs are not set");
  return mace->r_cut;
}

void PairSymmetrixMACE::init_style()
{
  if (atom->map_user == atom->MAP_NONE) error->all(FLERR, "symmetrix/mace requires 'atom_modify map [yes|array|hash]'");
  if (force->newton_pair == 0) error->all(FLERR, "symmetrix/mace requires newton pair on");
  if (mode == NO_MPI_MESSAGE_PASSING) {
    // ghosts of ghosts must be present: communication cutoff of at least two model cutoffs plus the skin
    const double need = 2.0 * mace->r_cut + neighbor->skin;
    if (comm->get_comm_cutoff() < need) {
      std::string value = std::to_string(need);
      char *args[2] = {(char *) "cutoff", const_cast<char *>(value.c_str())};
      comm->modify_params(2, args);
      if (comm->me == 0) utils::logmesg(lmp, "symmetrix/mace is setting the communication cutoff to {}\n", value);
    }
    neighbor->add_request(this, NeighConst::REQ_FULL | NeighConst::REQ_GHOST);
  } else {
    neighbor->add_request(this, NeighConst::REQ_FULL);
  }
}

/* ---------------------------------------------------------------------- */
// halo exchange of H1 / H1_adj rows (mpi_message_passing): one row of num_LM * num_channels doubles per atom

int PairSymmetrixMACE::pack_forward_comm(int n, int *list, double *buf, int /*pbc_flag*/, int * /*pbc*/)
{
  const int w = width();
  for (int q = 0; q < n; ++q) std::copy_n(&H1[(size_t) list[q] * w], w, buf + (size_t) q * w);
  return n * w;
}

void PairSymmetrixMACE::unpack_forward_comm(int n, int first, double *buf)
{
  const int w = width();
  std::copy_n(buf, (size_t) n * w, &H1[(size_t) first * w]);
}

int PairSymmetrixMACE::pack_reverse_comm(int n, int first, double *buf)
{
  const int w = width();
  std::copy_n(&H1_adj[(size_t) first * w], (size_t) n * w, buf);
  return n * w;
}

void PairSymmetrixMACE::unpack_reverse_comm(int n, int *list, double *buf)
{
  const int w = width();
  for (int q = 0; q < n; ++q)
    for (int k = 0; k < w; ++k) H1_adj[(size_t) list[q] * w + k] += buf[(size_t) q * w + k];
}

/* ---------------------------------------------------------------------- */
// The full neighbour list as flat edge arrays: pairs inside the model cutoff, receiver blocks in list order.
// Senders are named by atom row in neigh_j and, in neigh_indices, by the row of H1 the mode uses: the owner's node
// (no_domain_decomposition), the atom row itself (mpi_message_passing) or the node of the local / ghost atom
// (no_mpi_message_passing, where ghosts inside the cutoff of a local atom become nodes after the local ones).

void PairSymmetrixMACE::build_edges()
{
  const double rc2 = mace->r_cut * mace->r_cut;
  const int nall = atom->nlocal + atom->nghost;
  double **x = atom->x;
  const int inum = list->inum;
  edges.clear();
  edges.num_local_nodes = inum;
  node_of_atom.assign(nall, -1);
  for (int ii = 0; ii < inum; ++ii) node_of_atom[list->ilist[ii]] = ii;

  auto inside = [&](int i, int j, double *d) {
    d[0] = x[j][0] - x[i][0]; d[1] = x[j][1] - x[i][1]; d[2] = x[j][2] - x[i][2];
    return d[0] * d[0] + d[1] * d[1] + d[2] * d[2] < rc2;
  };
  std::vector<int> receivers(list->ilist, list->ilist + inum);
  if (mode == NO_MPI_MESSAGE_PASSING) {
    // ghosts within the cutoff of a local atom, in ascending atom row
    std::vector<char> wanted(nall, 0);
    double d[3];
    for (int ii = 0; ii < inum; ++ii) {
      const int i = list->ilist[ii];
      for (int jj = 0; jj < list->numneigh[i]; ++jj) {
        const int j = list->firstneigh[i][jj] & NEIGHMASK;
        if (node_of_atom[j] < 0 && inside(i, j, d)) wanted[j] = 1;
      }
    }
    for (int j = 0; j < nall; ++j)
      if (wanted[j]) { node_of_atom[j] = (int) receivers.size(); receivers.push_back(j); }
    edges.num_ghost_nodes = (int) receivers.size() - inum;
  }
  for (int i : receivers) {
    edges.node_i.push_back(i);
    edges.node_types.push_back(mace_types[atom->type[i] - 1]);
    int count = 0;
    double d[3];
    for (int jj = 0; jj < list->numneigh[i]; ++jj) {
      const int j = list->firstneigh[i][jj] & NEIGHMASK;
      if (!inside(i, j, d)) continue;
      ++count;
      int sender_atom = j, sender_row = j;
      if (mode == NO_DOMAIN_DECOMPOSITION) {
        sender_atom = atom->map(atom->tag[j]);          // periodic images fold onto their owners
        sender_row = node_of_atom[sender_atom];
      } else if (mode == NO_MPI_MESSAGE_PASSING) {
        // neighbours of a ghost node that are no nodes themselves only matter to layer 0, which does not read the row
        sender_row = std::max(node_of_atom[j], 0);
      }
      edges.neigh_j.push_back(sender_atom);
      edges.neigh_indices.push_back(sender_row);
      edges.neigh_types.push_back(mace_types[atom->type[j] - 1]);
      edges.xyz.insert(edges.xyz.end(), d, d + 3);
      edges.r.push_back(std::sqrt(d[0] * d[0] + d[1] * d[1] + d[2] * d[2]));
    }
    edges.num_neigh.push_back(count);
  }
}

void PairSymmetrixMACE::compute(int eflag, int vflag)
{
  ev_init(eflag, vflag);
  if (vflag_atom) error->all(FLERR, "Atomic virials not yet supported by pair_style symmetrix/mace.");
  build_edges();
  const int nall = atom->nlocal + atom->nghost;
  try {
    if (mode == NO_DOMAIN_DECOMPOSITION) {
      symmetrix_amd::evaluate_no_domain_decomposition(*mace, edges);
    } else if (mode == MPI_MESSAGE_PASSING) {
      symmetrix_amd::HaloExchange halo;
      halo.forward = [this](std::vector<double> &) { comm->forward_comm(this); };   // the buffers are this->H1 / H1_adj
      halo.reverse = [this](std::vector<double> &) { comm->reverse_comm(this); };
      symmetrix_amd::evaluate_mpi_message_passing(*mace, edges, nall, halo, H1, H1_adj);
    } else {
      symmetrix_amd::evaluate_no_mpi_message_passing(*mace, edges);
    }
    if (eflag_atom) eatom_nodes.assign(nall, 0.0);
    const double e = symmetrix_amd::total_energy(*mace, edges, eflag_atom ? eatom_nodes.data() : nullptr);
    if (eflag_global) eng_vdwl += e;
    if (eflag_atom)
      for (int i = 0; i < nall; ++i) eatom[i] += eatom_nodes[i];
    // f[i] -= f_ij, f[j] += f_ij and the virial, summed on the device in a fixed order; forces on ghost rows go back
    // to their owners with LAMMPS' reverse communication (newton pair on)
    if (nall > 0)   // an empty rank has no force array to point into
      symmetrix_amd::scatter_forces(*mace, edges, nall, &atom->f[0][0], vflag_global ? virial : nullptr);
  } catch (const std::exception &e) {
    error->one(FLERR, "symmetrix/mace: {}", e.what());
  }
}
