#include <cutile/cutile.hpp>
using namespace cutile;
int main() {
  cutile_testing_use_fake_hip;
  return 0;
}
