"""CPU oracle (checker) for the selective-scan hot path.  Test infrastructure only: the
shipped package never imports anything from here."""
